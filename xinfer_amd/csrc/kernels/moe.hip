// Routed experts (mixture of experts): the router, and the experts' products in a form that
// serves any sizes and both precisions, one (token, chosen expert) pair at a time.
//
//   router   z = Wr x + b in float32 (x may be the activation type's rounding of the stream);
//            the `top` experts with the largest z (ties: the lower index), their weights the
//            softmax over the chosen logits only; or (`all_scores`) the scores s = softmax(z) over
//            all experts, the chosen ones' divided by their sum + 1e-20.  Rows of Wr past the
//            experts' are further float32 products of the same x (a gate of a shared branch),
//            handed back as they are.
//   expert   y_e = Wd_e (act(Wg_e x) * (Wu_e x)), no biases; gate and up of all experts are stacked
//            [E, 2F, H] (gate rows first), down [E, H, F]; or without a gate, y_e = Wd_e act(Wu_e x)
//            with the up rows alone, [E, F, H].
//   output   sum over the chosen experts, in the order they were chosen, of weight * y_e: float32.
//   `scores` 2: the weights are sigmoid(z) of the chosen experts, as they are (the largest z are the largest scores).
//   A weight may instead multiply the expert's INPUT, y_e = expert(weight * x) (`in_wt` of the gate/up product: the
//   products are linear, so the weight multiplies their float32 sums before the activation; the down product then
//   gets weights of 1).
//
// Every sum runs in an order fixed by the sizes alone (lanes stride over k, then the wave's
// butterfly), so a token's result does not depend on the batch it is in.  The grouped
// matrix-core products for many tokens are in moe_mfma.hip; this file is the float32 path and
// what decode steps of few tokens use (a pair reads its expert's weights once: the least traffic
// there is when every pair has another expert).
#include "common.h"

namespace xi {

struct alignas(16) Bf8 { bf16 v[8]; };
constexpr int kRouteWaves = 4;
constexpr int kMaxExperts = 1024;
constexpr int kMaxTop = 64;

template <typename T>
__global__ __launch_bounds__(kRouteWaves* kWave) void moe_route_kernel(const T* __restrict__ x,
                                                                       const float* __restrict__ wr,
                                                                       const float* __restrict__ br, int* __restrict__ idx,
                                                                       float* __restrict__ wt, int H, int E, int top,
                                                                       int all_scores, float* __restrict__ extra, int X) {
  __shared__ float z[kMaxExperts];
  __shared__ float denom_all[2];
  __shared__ float chosen[kMaxTop];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const T* xr = x + (size_t)t * H;
  for (int e = wave; e < E + X; e += kRouteWaves) {
    const float* w = wr + (size_t)e * H;
    // four chains a lane, so that four rounds of loads are in flight; the order is fixed by H alone
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int k = lane;
    for (; k + 3 * kWave < H; k += 4 * kWave) {
      const float x0 = to_float(xr[k]), x1 = to_float(xr[k + kWave]), x2 = to_float(xr[k + 2 * kWave]),
                  x3 = to_float(xr[k + 3 * kWave]);
      const float w0 = w[k], w1 = w[k + kWave], w2 = w[k + 2 * kWave], w3 = w[k + 3 * kWave];
      a0 = fmaf(x0, w0, a0);
      a1 = fmaf(x1, w1, a1);
      a2 = fmaf(x2, w2, a2);
      a3 = fmaf(x3, w3, a3);
    }
    for (; k < H; k += kWave) a0 = fmaf(to_float(xr[k]), w[k], a0);
    float acc = wave_sum((a0 + a1) + (a2 + a3));
    if (lane == 0) {
      if (e < E) z[e] = acc + (br ? br[e] : 0.f);
      else extra[(size_t)t * X + (e - E)] = acc;
    }
  }
  __syncthreads();
  if (wave != 0) return;
  if (all_scores == 1) {     // the softmax's maximum and denominator over every expert, in a fixed order
    float m = -INFINITY;
    for (int e = lane; e < E; e += kWave) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float d = 0.f;
    for (int e = lane; e < E; e += kWave) d += expf(z[e] - m);
    d = wave_sum(d);
    if (lane == 0) {
      denom_all[0] = m;
      denom_all[1] = d;
    }
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
  }
  for (int r = 0; r < top; ++r) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += kWave)
      if (z[e] > best) {
        best = z[e];
        at = e;
      }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at >= E) at = E - 1;            // no finite logit left (rows of NaN): any valid expert
    if (lane == 0) {
      idx[(size_t)t * top + r] = at;
      chosen[r] = best;
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_s_waitcnt(0);      // lane 0's write to LDS is done before the wave reads z again
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0 && all_scores == 2) {
    for (int r = 0; r < top; ++r) wt[(size_t)t * top + r] = 1.f / (1.f + expf(-chosen[r]));
  } else if (lane == 0 && all_scores) {
    const float m = denom_all[0], d = denom_all[1];
    float sum = 0.f;
    for (int r = 0; r < top; ++r) sum += expf(chosen[r] - m) / d;
    for (int r = 0; r < top; ++r) wt[(size_t)t * top + r] = (expf(chosen[r] - m) / d) / (sum + 1e-20f);
  } else if (lane == 0) {
    const float m = chosen[0];
    float sum = 0.f;
    for (int r = 0; r < top; ++r) sum += expf(chosen[r] - m);
    for (int r = 0; r < top; ++r) wt[(size_t)t * top + r] = expf(chosen[r] - m) / sum;
  }
}

template <int ACT>
__device__ __forceinline__ float moe_act(float z) {
  if constexpr (ACT == 0) return z / (1.f + expf(-z));
  else if constexpr (ACT == 2) return z > 0.f ? z * z : 0.f;      // the square of relu
  else return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// One workgroup: a pair (token, rank) and FT features of its expert; the token's row sits in LDS.
constexpr int kMoeWaves = 4;
// GATED false: the weights hold the up rows alone, [E, F, H], and mid = act(up).
template <typename T, int ACT, bool GATED>
__global__ __launch_bounds__(kMoeWaves* kWave) void moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ wgu,
                                                                       const int* __restrict__ idx, T* __restrict__ mid,
                                                                       int H, int F, int top, int FT,
                                                                       const float* __restrict__ in_wt) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x, t = pair / top;
  const int e = idx[pair];
  const float wi = in_wt ? in_wt[pair] : 1.f;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  for (int k = threadIdx.x; k < H; k += blockDim.x) xs[k] = to_float(x[(size_t)t * H + k]);
  __syncthreads();
  const T* wg = wgu + (size_t)e * (GATED ? 2 : 1) * F * H;
  const int f_end = min(F, (int)(blockIdx.y + 1) * FT);
  for (int f = blockIdx.y * FT + wave; f < f_end; f += kMoeWaves) {
    const T* g = wg + (size_t)f * H;
    const T* u = GATED ? wg + (size_t)(F + f) * H : g;
    float ag = 0.f, au = 0.f;
    if constexpr (sizeof(T) == 2) {
      if (H % 8 == 0) {              // 16 bytes a lane and load; the order of a sum is still fixed by H alone
        for (int k = 8 * lane; k < H; k += 8 * kWave) {
          const Bf8 gv = *reinterpret_cast<const Bf8*>(g + k);
          Bf8 uv;
          if constexpr (GATED) uv = *reinterpret_cast<const Bf8*>(u + k);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            ag = fmaf(to_float(gv.v[e]), xs[k + e], ag);
            if constexpr (GATED) au = fmaf(to_float(uv.v[e]), xs[k + e], au);
          }
        }
      } else {
        for (int k = lane; k < H; k += kWave) {
          ag = fmaf(to_float(g[k]), xs[k], ag);
          if constexpr (GATED) au = fmaf(to_float(u[k]), xs[k], au);
        }
      }
    } else {
      for (int k = lane; k < H; k += kWave) {
        ag = fmaf(to_float(g[k]), xs[k], ag);
        if constexpr (GATED) au = fmaf(to_float(u[k]), xs[k], au);
      }
    }
    ag = wave_sum(ag) * wi;
    if constexpr (GATED) au = wave_sum(au) * wi;
    if (lane == 0) mid[(size_t)pair * F + f] = from_float<T>(GATED ? moe_act<ACT>(ag) * au : moe_act<ACT>(ag));
  }
}

// One workgroup: a token and NTile output features; the token's `top` rows of mid sit in LDS.
template <typename T>
__global__ __launch_bounds__(kMoeWaves* kWave) void moe_down_kernel(const T* __restrict__ mid, const T* __restrict__ wd,
                                                                    const int* __restrict__ idx, const float* __restrict__ wt,
                                                                    float* __restrict__ out, int H, int F, int top, int NTile) {
  extern __shared__ float ms[];       // [top, F]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  for (int i = threadIdx.x; i < top * F; i += blockDim.x) ms[i] = to_float(mid[(size_t)t * top * F + i]);
  __syncthreads();
  const int n_end = min(H, (int)(blockIdx.y + 1) * NTile);
  for (int n = blockIdx.y * NTile + wave; n < n_end; n += kMoeWaves) {
    float total = 0.f;
    for (int r = 0; r < top; ++r) {
      const T* w = wd + ((size_t)idx[(size_t)t * top + r] * H + n) * F;
      float acc = 0.f;
      if (sizeof(T) == 2 && F % 8 == 0) {
        for (int f = 8 * lane; f < F; f += 8 * kWave) {
          const Bf8 wv = *reinterpret_cast<const Bf8*>(w + f);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc = fmaf(to_float(wv.v[e]), ms[r * F + f + e], acc);
        }
      } else {
        for (int f = lane; f < F; f += kWave) acc = fmaf(to_float(w[f]), ms[r * F + f], acc);
      }
      acc = wave_sum(acc);
      total += wt[(size_t)t * top + r] * acc;
    }
    if (lane == 0) out[(size_t)t * H + n] = total;
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// x [T, H] in `dtype`; wr float32 [E, H]; br float32 [E] or null; idx int32 [T, top]; wt float32 [T, top].
// all_scores: 0, 1 (see the head of the file) or 2 (sigmoid of the chosen logits).  extra float32 [T, X]: the products with rows E .. E + X - 1 of wr (X may be 0).
int xi_moe_route(const void* x, int dtype, const float* wr, const float* br, int* idx, float* wt, int n_tok, int H, int E,
                 int top, int all_scores, float* extra, int X, hipStream_t stream) {
  XI_CHECK(X >= 0 && (X == 0 || extra != nullptr), "moe_route: %d further rows need a place for their results", X);
  XI_CHECK(n_tok >= 0 && H > 0 && E > 0 && E <= kMaxExperts, "moe_route: bad sizes T=%d H=%d experts=%d (at most %d)", n_tok,
           H, E, kMaxExperts);
  XI_CHECK(all_scores >= 0 && all_scores <= 2, "moe_route: unknown kind of scores %d", all_scores);
  XI_CHECK(top > 0 && top <= E && top <= kMaxTop, "moe_route: %d of %d experts cannot be chosen (at most %d)", top, E, kMaxTop);
  if (n_tok == 0) return 0;
  if (dtype == kF32)
    moe_route_kernel<float><<<n_tok, kRouteWaves * kWave, 0, stream>>>((const float*)x, wr, br, idx, wt, H, E, top, all_scores,
                                                                       extra, X);
  else if (dtype == kBF16)
    moe_route_kernel<bf16><<<n_tok, kRouteWaves * kWave, 0, stream>>>((const bf16*)x, wr, br, idx, wt, H, E, top, all_scores,
                                                                      extra, X);
  else
    XI_CHECK(false, "moe_route: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("moe_route");
  return 0;
}

// x [T, H], wgu [E, 2F, H], idx [T * top] -> mid [T * top, F] = act(gate) * up, all in `dtype`;
// gated 0: wgu [E, F, H] and mid = act(up).  act: 0 silu, 1 gelu (tanh form), 2 the square of relu.
// in_wt float32 [T * top] or null: a weight a pair on the expert's input.
int xi_moe_gate_up(const void* x, const void* wgu, const int* idx, void* mid, int dtype, int act, int gated, int n_tok, int H,
                   int F, int E, int top, const float* in_wt, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && F > 0 && E > 0 && top > 0, "moe_gate_up: bad sizes T=%d H=%d F=%d E=%d top=%d", n_tok, H, F, E,
           top);
  XI_CHECK(act >= 0 && act <= 2, "moe_gate_up: unknown activation %d", act);
  XI_CHECK((size_t)H * sizeof(float) <= 64 * 1024, "moe_gate_up: a row of %d does not fit in LDS", H);
  if (n_tok == 0) return 0;
  const long long pairs = (long long)n_tok * top;
  XI_CHECK(pairs < (1ll << 31), "moe_gate_up: too many tokens");
  const int FT = 64;
  dim3 grid((unsigned)pairs, (unsigned)((F + FT - 1) / FT));
  XI_CHECK(grid.y <= 65535u, "moe_gate_up: F=%d is too large", F);
  const size_t lds = (size_t)H * sizeof(float);
#define XI_GU(TT, A, G)                                                                                         \
  do {                                                                                                          \
    auto kern = moe_gate_up_kernel<TT, A, G>;                                                                   \
    if (lds > 48 * 1024) {                                                                                      \
      hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      XI_CHECK(e_ == hipSuccess, "moe_gate_up: cannot get %zu bytes of LDS", lds);                              \
    }                                                                                                           \
    kern<<<grid, kMoeWaves * kWave, lds, stream>>>((const TT*)x, (const TT*)wgu, idx, (TT*)mid, H, F, top, FT, in_wt); \
  } while (0)
#define XI_GU_A(TT, G)            \
  do {                            \
    if (act == 0) XI_GU(TT, 0, G); \
    else if (act == 1) XI_GU(TT, 1, G); \
    else XI_GU(TT, 2, G);         \
  } while (0)
  if (dtype == kF32 && gated) XI_GU_A(float, true);
  else if (dtype == kF32) XI_GU_A(float, false);
  else if (dtype == kBF16 && gated) XI_GU_A(bf16, true);
  else if (dtype == kBF16) XI_GU_A(bf16, false);
  else XI_CHECK(false, "moe_gate_up: unknown dtype %d", dtype);
#undef XI_GU_A
#undef XI_GU
  XI_LAUNCH_CHECK("moe_gate_up");
  return 0;
}

// mid [T * top, F], wd [E, H, F] in `dtype`; idx, wt [T, top] -> out float32 [T, H].
int xi_moe_down(const void* mid, const void* wd, const int* idx, const float* wt, float* out, int dtype, int n_tok, int H,
                int F, int E, int top, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && F > 0 && E > 0 && top > 0, "moe_down: bad sizes T=%d H=%d F=%d E=%d top=%d", n_tok, H, F, E, top);
  const size_t lds = (size_t)top * F * sizeof(float);
  XI_CHECK(lds <= 64 * 1024, "moe_down: %d rows of %d do not fit in LDS", top, F);
  if (n_tok == 0) return 0;
  const int NTile = 64;
  dim3 grid((unsigned)n_tok, (unsigned)((H + NTile - 1) / NTile));
  XI_CHECK(grid.y <= 65535u, "moe_down: H=%d is too large", H);
#define XI_DN(TT)                                                                                               \
  do {                                                                                                          \
    auto kern = moe_down_kernel<TT>;                                                                            \
    if (lds > 48 * 1024) {                                                                                      \
      hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      XI_CHECK(e_ == hipSuccess, "moe_down: cannot get %zu bytes of LDS", lds);                                 \
    }                                                                                                           \
    kern<<<grid, kMoeWaves * kWave, lds, stream>>>((const TT*)mid, (const TT*)wd, idx, wt, out, H, F, top, NTile); \
  } while (0)
  if (dtype == kF32) XI_DN(float);
  else if (dtype == kBF16) XI_DN(bf16);
  else XI_CHECK(false, "moe_down: unknown dtype %d", dtype);
#undef XI_DN
  XI_LAUNCH_CHECK("moe_down");
  return 0;
}

}  // extern "C"
