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
  if (dtype == kF32)
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
