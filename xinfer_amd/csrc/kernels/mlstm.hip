// What stands around the state of a matrix memory (mLSTM): the gates in front of it and the normalizer,
// the heads' norm and the output gate behind it.  The state itself, S <- keep S + take k v^T with the sum of the
// weighted keys n as one more value column, is walked by `linear_scan_kernel` (recurrence.hip, `gates`).
//
// `mlstm_gates_kernel`: per request and head, from the logits zi, zf (float32 columns of a product, plus a bias)
//     log_in = cap tanh((zi + bi) / cap)          log_keep = logsigmoid(cap tanh((zf + bf) / cap))
//     m' = max(log_keep + m, log_in)             (m: a running maximum, state of the request, 0 when it starts)
//     keep = exp(log_keep + m - m')   take = exp(log_in - m')   floor = exp(-m')
// and writes (keep, take) [T, H, 2] and floor [T, H].  The chain over m is two operations a token and is walked by
// one wave, 64 tokens' gates in its lanes' registers at a time; logits before and exponentials after are made by the
// whole workgroup, a block of tokens at a time.
// Everything float32: what a token gets does not depend on how the prompt was cut, bit for bit.
//
// `mlstm_finish_kernel`: o [T, H, dv + 1] float32 (the state's results; the last column is n . q):
//     y = o[:dv] / (max(|o[dv]|, floor) + 1e-6);  y / sqrt(mean(y^2) + eps) * w[h, :] * sigmoid(g[t, h, :])
// rounded to the activation type for the output projection.  One wave per (token, head).
#include "common.h"

namespace xi {

constexpr int kGateBlock = 1024;     // tokens a round: the chain of a round runs while nothing else does, so rounds are few

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__global__ __launch_bounds__(kGateBlock) void mlstm_gates_kernel(const float* __restrict__ z, long long z_stride,
                                                                 const float* __restrict__ bias, float cap,
                                                                 float* __restrict__ m_state, long long slot_stride,
                                                                 const long long* __restrict__ slots,
                                                                 const int* __restrict__ cu_q, float* __restrict__ gates,
                                                                 float* __restrict__ floor_out, int H) {
  __shared__ float li[kGateBlock], lk[kGateBlock], ms[kGateBlock + 1];
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  if (t1 <= t0) return;
  float* mp = m_state + (size_t)slots[b] * slot_stride + h;
  const float bi = bias[h], bf = bias[H + h], inv_cap = 1.f / cap;
  if (threadIdx.x == 0) ms[0] = *mp;
  for (int base = t0; base < t1; base += kGateBlock) {
    const int n = min(kGateBlock, t1 - base);
    const int t = base + threadIdx.x;
    if (threadIdx.x < n) {
      const float* zr = z + (size_t)t * z_stride;
      li[threadIdx.x] = cap * tanhf((zr[h] + bi) * inv_cap);
      lk[threadIdx.x] = log_sigmoid(cap * tanhf((zr[H + h] + bf) * inv_cap));
    }
    __syncthreads();
    if (threadIdx.x < kWave) {           // the first wave walks the chain: lane l holds token l's gates of a run of 64, every
      float m = ms[0];                   // lane follows the whole chain (the gates reach it from the lanes' registers, not
      for (int first = 0; first < n; first += kWave) {     // from memory) and keeps its own token's value
        const int i = first + (int)threadIdx.x;
        const int keep_bits = __float_as_int(i < n ? lk[i] : 0.f);            // past the end: m stays what it is
        const int in_bits = __float_as_int(i < n ? li[i] : -INFINITY);
        float mine = 0.f;
#pragma unroll
        for (int e = 0; e < kWave; ++e) {
          m = fmaxf(__int_as_float(__builtin_amdgcn_readlane(keep_bits, e)) + m, __int_as_float(__builtin_amdgcn_readlane(in_bits, e)));
          if ((int)threadIdx.x == e) mine = m;
        }
        if (i < n) ms[i + 1] = mine;
      }
    }
    __syncthreads();
    if (threadIdx.x < n) {
      const float m_old = ms[threadIdx.x], m_new = ms[threadIdx.x + 1];
      float* g = gates + ((size_t)t * H + h) * 2;
      g[0] = expf(lk[threadIdx.x] + m_old - m_new);
      g[1] = expf(li[threadIdx.x] - m_new);
      floor_out[(size_t)t * H + h] = expf(-m_new);
    }
    __syncthreads();
    if (threadIdx.x == 0) ms[0] = ms[n];
    // (thread 0 alone reads ms[0] before the next barrier)
  }
  if (threadIdx.x == 0) *mp = ms[0];
}

template <typename T>
__global__ __launch_bounds__(256) void mlstm_finish_kernel(const float* __restrict__ o, const float* __restrict__ floor_in,
                                                           const float* __restrict__ w, float eps, const T* __restrict__ g,
                                                           long long g_stride, T* __restrict__ out, long long pairs, int H,
                                                           int dv) {
  const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long long t = pair / H;
  const int h = (int)(pair - t * H);
  const float* x = o + (size_t)pair * (dv + 1);
  const float inv_den = 1.f / (fmaxf(fabsf(x[dv]), floor_in[pair]) + 1e-6f);
  float ss = 0.f;
  for (int i = lane; i < dv; i += kWave) {
    const float y = x[i] * inv_den;
    ss = fmaf(y, y, ss);
  }
  const float inv = rsqrtf(wave_sum(ss) / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + (size_t)h * dv;
  const float* wr = w + (size_t)h * dv;
  T* orow = out + (size_t)pair * dv;
  for (int i = lane; i < dv; i += kWave) {
    const float gv = to_float(gr[i]);
    orow[i] = from_float<T>((x[i] * inv_den) * inv * wr[i] * (1.f / (1.f + expf(-gv))));
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// z float32 rows of z_stride floats: columns 0 .. H-1 the input gate's logits, H .. 2H-1 the forget gate's; bias float32
// [2 H]; m_state float32, slot s at m_state + s * slot_stride, H floats; slots int64 [B]; cu_q int32 [B + 1];
// gates float32 [T, H, 2]; floor_out float32 [T, H].
int xi_mlstm_gates(const float* z, long long z_stride, const float* bias, float cap, float* m_state, long long slot_stride,
                   const long long* slots, const int* cu_q, float* gates, float* floor_out, int n_seqs, int H,
                   hipStream_t stream) {
  XI_CHECK(n_seqs >= 0 && H > 0 && H <= 65535 && z_stride >= 2 * (long long)H && slot_stride >= H,
           "mlstm_gates: bad sizes B=%d H=%d", n_seqs, H);
  XI_CHECK(cap > 0.f, "mlstm_gates: the gates' cap must be positive, got %g", (double)cap);
  if (n_seqs == 0) return 0;
  mlstm_gates_kernel<<<dim3((unsigned)n_seqs, (unsigned)H), kGateBlock, 0, stream>>>(z, z_stride, bias, cap, m_state, slot_stride,
                                                                                    slots, cu_q, gates, floor_out, H);
  XI_LAUNCH_CHECK("mlstm_gates");
  return 0;
}

// o float32 [T, H, dv + 1]; floor_in float32 [T, H]; w float32 [H dv]; g rows of g_stride elements holding [H dv]
// gates in `dtype`; out [T, H dv] in `dtype`.
int xi_mlstm_finish(const float* o, const float* floor_in, const float* w, float eps, const void* g, long long g_stride,
                    void* out, int dtype, int n_tok, int H, int dv, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && dv > 0 && g_stride >= (long long)H * dv, "mlstm_finish: bad sizes T=%d H=%d dv=%d", n_tok, H, dv);
  if (n_tok == 0) return 0;
  const long long pairs = (long long)n_tok * H;
  const long long blocks = (pairs + 3) / 4;
  XI_CHECK(blocks < (1ll << 31), "mlstm_finish: too many tokens");
  if (dtype == kF32)
    mlstm_finish_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(o, floor_in, w, eps, (const float*)g, g_stride, (float*)out,
                                                                     pairs, H, dv);
  else if (dtype == kBF16)
    mlstm_finish_kernel<bf16><<<(unsigned)blocks, 256, 0, stream>>>(o, floor_in, w, eps, (const bf16*)g, g_stride, (bf16*)out,
                                                                    pairs, H, dv);
  else
    XI_CHECK(false, "mlstm_finish: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("mlstm_finish");
  return 0;
}

}  // extern "C"
