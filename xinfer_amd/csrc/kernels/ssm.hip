// What stands around the state of a selective state-space mixer: the short causal convolution in front of it
// and the gate and grouped norm behind it.
//
// `causal_conv_kernel`: C channels of a packed projection (columns from an offset), each with its own `taps`
// weights (w [C, taps], w[c, taps - 1 - k] for the input k tokens back) and a bias; out[t, c] = silu(bias[c] + sum_j w[c, j]
// u[t - (taps - 1) + j, c]), where inputs from before the step's portion are the request's tail (the last taps - 1
// inputs of earlier steps, float32 [slots, taps - 1, C], oldest first; zeros for a request's first tokens: a slot
// is cleared when its request starts).  Sums in float32, one rounding.
// `conv_tail_kernel` then moves the tail on by the step's tokens (a launch of its own: the tail is read by the
// portion's first tokens and written from its last, which other workgroups hold).
//
// `gated_group_norm_kernel`: v = (y + D[h] x) * silu(z); each of `groups` equal parts of a token's row divided by
// its own root mean square (eps inside the root), times a weight as long as the row; y float32 [T, heads, dv] (the
// state's results), x and z columns of packed rows.  All float32 until the one rounding of the store.
#include "common.h"

namespace xi {

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ u, long long u_stride,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          const float* __restrict__ tails, long long slot_stride,
                                                          const long long* __restrict__ slots,
                                                          const int* __restrict__ tok_seq, const int* __restrict__ cu_q,
                                                          T* __restrict__ out, int C, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = tok_seq[t];
  const int t0 = cu_q[b];
  const float* tail = tails + (size_t)slots[b] * slot_stride;
  float acc = bias[c];
  for (int j = 0; j < taps; ++j) {
    const int s = t - (taps - 1) + j;
    // before the portion: s = t0 - k, k = 1 .. taps - 1, the tail's entry taps - 1 - k
    const float x = s >= t0 ? to_float(u[(size_t)s * u_stride + c]) : tail[(size_t)(taps - 1 - (t0 - s)) * C + c];
    acc = fmaf(w[(size_t)c * taps + j], x, acc);
  }
  out[(size_t)t * C + c] = from_float<T>(acc / (1.f + expf(-acc)));
}

template <typename T>
__global__ __launch_bounds__(256) void conv_tail_kernel(const T* __restrict__ u, long long u_stride,
                                                        float* __restrict__ tails, long long slot_stride,
                                                        const long long* __restrict__ slots, const int* __restrict__ cu_q,
                                                        int C, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  const int n = t1 - t0;
  if (n <= 0) return;
  float* tail = tails + (size_t)slots[b] * slot_stride;
  // entry i of the new tail is the input taps - 1 - i tokens before the end; an entry that is older than the
  // portion is entry i + n of the old tail, which this thread has not overwritten yet (i ascends)
  for (int i = 0; i < taps - 1; ++i) {
    const int s = t1 - (taps - 1) + i;
    tail[(size_t)i * C + c] = s >= t0 ? to_float(u[(size_t)s * u_stride + c]) : tail[(size_t)(i + n) * C + c];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ x,
                                                               long long x_stride, const float* __restrict__ skip,
                                                               const T* __restrict__ z, long long z_stride,
                                                               const float* __restrict__ w, float eps, T* __restrict__ out,
                                                               int width, int dv, int groups) {
  __shared__ float scratch[4];
  const int t = blockIdx.x, g = blockIdx.y;
  const int per = width / groups;
  const int lo = g * per;
  const float* yr = y + (size_t)t * width;
  const T* xr = x + (size_t)t * x_stride;
  const T* zr = z + (size_t)t * z_stride;
  auto value = [&](int i) {
    const float zv = to_float(zr[i]);
    return fmaf(skip[i / dv], to_float(xr[i]), yr[i]) * (zv / (1.f + expf(-zv)));
  };
  float ss = 0.f;
  for (int i = lo + threadIdx.x; i < lo + per; i += blockDim.x) {
    const float v = value(i);
    ss = fmaf(v, v, ss);
  }
  const float inv = rsqrtf(block_sum<4>(ss, scratch) / (float)per + eps);
  for (int i = lo + threadIdx.x; i < lo + per; i += blockDim.x)
    out[(size_t)t * width + i] = from_float<T>(value(i) * inv * w[i]);
}

// ---- eight channels a thread ------------------------------------------------------------------------------------
// Rows whose channels come in whole 16-byte chunks: a thread takes 8 channels side by side, one load a row.
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float (&v)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const unsigned u[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(u[i] << 16);
    v[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float (&v)[8]) {
  unsigned u[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16 lo = __float2bfloat16(v[2 * i]), hi = __float2bfloat16(v[2 * i + 1]);
    u[i] = (unsigned)*reinterpret_cast<const unsigned short*>(&lo) | ((unsigned)*reinterpret_cast<const unsigned short*>(&hi) << 16);
  }
  *reinterpret_cast<uint4*>(p) = make_uint4(u[0], u[1], u[2], u[3]);
}

// The convolution for a thread's 8 channels over a run of `run` tokens: the last TAPS - 1 inputs stay in registers
// from token to token, so a row of u is read once; at a run's first token they come from the rows before (or the
// request's tail), at a sequence's first token from its tail.  The sums are those of `causal_conv_kernel`, term by term.
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_run_kernel(const T* __restrict__ u, long long u_stride,
                                                              const float* __restrict__ w, const float* __restrict__ bias,
                                                              const float* __restrict__ tails, long long slot_stride,
                                                              const long long* __restrict__ slots,
                                                              const int* __restrict__ tok_seq, const int* __restrict__ cu_q,
                                                              T* __restrict__ out, int n_tok, int C, int run) {
  const int c = 8 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c >= C) return;
  const int ta = blockIdx.x * run;
  const int tb = ta + run < n_tok ? ta + run : n_tok;
  float wt[TAPS][8], bs[8], win[TAPS > 1 ? TAPS - 1 : 1][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    bs[i] = bias[c + i];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wt[j][i] = w[(size_t)(c + i) * TAPS + j];
  }
  int b = -1, t0 = 0;
  for (int t = ta; t < tb; ++t) {
    const int bt = tok_seq[t];
    if (bt != b) {                                   // the run's first token, or a sequence's
      b = bt;
      t0 = cu_q[b];
      const float* tail = tails + (size_t)slots[b] * slot_stride;
#pragma unroll
      for (int i = 0; i < TAPS - 1; ++i) {
        const int s = t - (TAPS - 1) + i;
        if (s >= t0) load8(u + (size_t)s * u_stride + c, win[i]);
        else load8(tail + (size_t)(TAPS - 1 - (t0 - s)) * C + c, win[i]);
      }
    }
    float cur[8], o[8];
    load8(u + (size_t)t * u_stride + c, cur);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float acc = bs[i];
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) acc = fmaf(wt[j][i], win[j][i], acc);
      acc = fmaf(wt[TAPS - 1][i], cur[i], acc);
      o[i] = acc / (1.f + expf(-acc));
    }
    store8(out + (size_t)t * C + c, o);
#pragma unroll
    for (int j = 0; j + 1 < TAPS - 1; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) win[j][i] = win[j + 1][i];
    if (TAPS > 1) {
#pragma unroll
      for (int i = 0; i < 8; ++i) win[TAPS > 1 ? TAPS - 2 : 0][i] = cur[i];
    }
  }
}

// The gate and the norm for rows in whole chunks of 8 that lie within one head: a thread's first kGnKeep chunks stay
// in registers between the sum of squares and the store.
constexpr int kGnKeep = 4;
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_vec_kernel(const float* __restrict__ y, const T* __restrict__ x,
                                                                   long long x_stride, const float* __restrict__ skip,
                                                                   const T* __restrict__ z, long long z_stride,
                                                                   const float* __restrict__ w, float eps,
                                                                   T* __restrict__ out, int width, int dv, int groups) {
  __shared__ float scratch[4];
  const int t = blockIdx.x, g = blockIdx.y;
  const int per = width / groups;
  const int lo = g * per;
  const float* yr = y + (size_t)t * width;
  const T* xr = x + (size_t)t * x_stride;
  const T* zr = z + (size_t)t * z_stride;
  auto values = [&](int i, float (&v)[8]) {
    float yv[8], xv[8], zv[8];
    load8(yr + i, yv);
    load8(xr + i, xv);
    load8(zr + i, zv);
    const float sk = skip[i / dv];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = fmaf(sk, xv[e], yv[e]) * (zv[e] / (1.f + expf(-zv[e])));
  };
  float kept[kGnKeep][8];
  float ss = 0.f;
  int n = 0;
  for (int i = lo + 8 * threadIdx.x; i < lo + per; i += 8 * blockDim.x, ++n) {
    float v[8];
    values(i, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(v[e], v[e], ss);
#pragma unroll
    for (int k = 0; k < kGnKeep; ++k)
      if (k == n) {
#pragma unroll
        for (int e = 0; e < 8; ++e) kept[k][e] = v[e];
      }
  }
  const float inv = rsqrtf(block_sum<4>(ss, scratch) / (float)per + eps);
  n = 0;
  for (int i = lo + 8 * threadIdx.x; i < lo + per; i += 8 * blockDim.x, ++n) {
    float v[8], wv[8];
    if (n < kGnKeep) {
#pragma unroll
      for (int k = 0; k < kGnKeep; ++k)
        if (k == n) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = kept[k][e];
        }
    } else {
      values(i, v);
    }
    load8(w + i, wv);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = v[e] * inv * wv[e];
    store8(out + (size_t)t * width + i, v);
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// u: rows of u_stride elements whose first C (from the given pointer) are the channels; w float32 [C, taps], bias
// float32 [C]; tails float32, slot s at tails + s * slot_stride, [taps - 1, C] each; slots int64 [B]; tok_seq int32 [T];
// cu_q int32 [B + 1]; out [T, C] in `dtype`.
int xi_causal_conv(const void* u, long long u_stride, int dtype, const float* w, const float* bias, const float* tails,
                   long long slot_stride, const long long* slots, const int* tok_seq, const int* cu_q, void* out, int n_tok,
                   int C, int taps, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && C > 0 && taps >= 1 && u_stride >= C, "causal_conv: bad sizes T=%d C=%d taps=%d", n_tok, C, taps);
  XI_CHECK(slot_stride >= (long long)(taps - 1) * C, "causal_conv: a slot's tail is too small");
  if (n_tok == 0) return 0;
  // channels in whole 16-byte chunks and few taps: eight channels a thread, runs of tokens where there are many
  const size_t esize = dtype == kF32 ? 4 : 2;
  if ((dtype == kF32 || dtype == kBF16) && taps <= 5 && C % 8 == 0 && u_stride % 8 == 0 && slot_stride % 4 == 0 &&
      (reinterpret_cast<uintptr_t>(u) & 15) == 0 && (reinterpret_cast<uintptr_t>(tails) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 15) == 0 && esize) {
    const int run = n_tok >= 1024 ? 8 : n_tok >= 256 ? 4 : 1;
    dim3 vgrid((unsigned)((n_tok + run - 1) / run), (unsigned)((C / 8 + 255) / 256));
#define XI_CONV_RUN(TT, TAPS)                                                                                          \
  causal_conv_run_kernel<TT, TAPS><<<vgrid, 256, 0, stream>>>((const TT*)u, u_stride, w, bias, tails, slot_stride, slots, \
                                                             tok_seq, cu_q, (TT*)out, n_tok, C, run)
#define XI_CONV_TAPS(TT)              \
  switch (taps) {                     \
    case 1: XI_CONV_RUN(TT, 1); break; \
    case 2: XI_CONV_RUN(TT, 2); break; \
    case 3: XI_CONV_RUN(TT, 3); break; \
    case 4: XI_CONV_RUN(TT, 4); break; \
    default: XI_CONV_RUN(TT, 5); break; \
  }
    if (dtype == kF32) {
      XI_CONV_TAPS(float)
    } else {
      XI_CONV_TAPS(bf16)
    }
#undef XI_CONV_TAPS
#undef XI_CONV_RUN
    XI_LAUNCH_CHECK("causal_conv");
    return 0;
  }
  dim3 grid((unsigned)n_tok, (unsigned)((C + 255) / 256));
  XI_CHECK(grid.y <= 65535u, "causal_conv: too many channels");
  if (dtype == kF32)
    causal_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, u_stride, w, bias, tails, slot_stride, slots, tok_seq,
                                                        cu_q, (float*)out, C, taps);
  else if (dtype == kBF16)
    causal_conv_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)u, u_stride, w, bias, tails, slot_stride, slots, tok_seq,
                                                       cu_q, (bf16*)out, C, taps);
  else
    XI_CHECK(false, "causal_conv: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("causal_conv");
  return 0;
}

int xi_conv_tail(const void* u, long long u_stride, int dtype, float* tails, long long slot_stride, const long long* slots,
                 const int* cu_q, int n_seqs, int C, int taps, hipStream_t stream) {
  XI_CHECK(n_seqs >= 0 && C > 0 && taps >= 1 && u_stride >= C, "conv_tail: bad sizes B=%d C=%d taps=%d", n_seqs, C, taps);
  XI_CHECK(slot_stride >= (long long)(taps - 1) * C, "conv_tail: a slot's tail is too small");
  if (n_seqs == 0 || taps == 1) return 0;
  dim3 grid((unsigned)n_seqs, (unsigned)((C + 255) / 256));
  XI_CHECK(grid.y <= 65535u, "conv_tail: too many channels");
  if (dtype == kF32)
    conv_tail_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, u_stride, tails, slot_stride, slots, cu_q, C, taps);
  else if (dtype == kBF16)
    conv_tail_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)u, u_stride, tails, slot_stride, slots, cu_q, C, taps);
  else
    XI_CHECK(false, "conv_tail: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("conv_tail");
  return 0;
}

// y float32 [T, width]; x, z rows of x_stride / z_stride elements with `width` columns from the given pointers, in
// `dtype`; skip float32 [width / dv]; w float32 [width]; out [T, width] in `dtype`.
int xi_gated_group_norm(const float* y, const void* x, long long x_stride, const float* skip, const void* z,
                        long long z_stride, const float* w, float eps, void* out, int dtype, int n_tok, int width, int dv,
                        int groups, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && width > 0 && dv > 0 && groups > 0 && width % dv == 0 && width % groups == 0,
           "gated_group_norm: bad sizes T=%d width=%d dv=%d groups=%d", n_tok, width, dv, groups);
  XI_CHECK(x_stride >= width && z_stride >= width, "gated_group_norm: the rows are too short");
  XI_CHECK(groups <= 65535, "gated_group_norm: too many groups");
  if (n_tok == 0) return 0;
  dim3 grid((unsigned)n_tok, (unsigned)groups);
  const bool chunks = (width / groups) % 8 == 0 && dv % 8 == 0 && x_stride % 8 == 0 && z_stride % 8 == 0 &&
                      (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(z) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(y) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (chunks && dtype == kF32) {
    gated_group_norm_vec_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)x, x_stride, skip, (const float*)z, z_stride,
                                                                 w, eps, (float*)out, width, dv, groups);
  } else if (chunks && dtype == kBF16) {
    gated_group_norm_vec_kernel<bf16><<<grid, 256, 0, stream>>>(y, (const bf16*)x, x_stride, skip, (const bf16*)z, z_stride, w,
                                                                eps, (bf16*)out, width, dv, groups);
  } else if (dtype == kF32)
    gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)x, x_stride, skip, (const float*)z, z_stride, w,
                                                             eps, (float*)out, width, dv, groups);
  else if (dtype == kBF16)
    gated_group_norm_kernel<bf16><<<grid, 256, 0, stream>>>(y, (const bf16*)x, x_stride, skip, (const bf16*)z, z_stride, w, eps,
                                                            (bf16*)out, width, dv, groups);
  else
    XI_CHECK(false, "gated_group_norm: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("gated_group_norm");
  return 0;
}

}  // extern "C"
