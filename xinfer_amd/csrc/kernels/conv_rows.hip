// A packed projection row [q (nq d) | k (nkv d) | v (nkv dv)] made ready for an attention whose q, k and v pass a
// short causal convolution and whose heads' scores are mixed, in one kernel a token:
//
//   convolution   y_t[c] = sum_j w[c, j] u_(t - taps + 1 + j)[c] per channel over the last `taps` tokens (w float32
//                 [C, taps], no bias, no activation); inputs from before the step's portion come from the request's
//                 tail (the last taps - 1 projected rows of earlier steps, float32 [slots, taps - 1, C], oldest first;
//                 zeros for a request's first tokens).  `conv_tail_kernel` (ssm.hip) moves the tail on afterwards.
//                 One tap is a factor a channel and needs no tail; no weights: no convolution.
//   norms         RMS norm over the WHOLE q part and the whole k part (one mean over all heads, weights qw [nq d] and
//                 kw [nkv d]; null: none); with `v_unit` every value head divided by its own root mean square over dv;
//                 eps inside the roots.
//   mixed heads   with `talk` T float32 [nq, nq], head h's score of a key is sum_g T[h, g] (q_g . k_kv(g)).  The sum
//                 moves to the query's side: q'_h = [sum_{g in group c} T[h, g] q_g for every kv head c], nkv d dims,
//                 which is scored against the token's WHOLE k row.  q_out is then [T, nq, nkv d] and the K pool holds
//                 one head of nkv d dims a token, [pages, 1, page, nkv d] (the same bytes as a row of k); without
//                 `talk` q_out is [T, nq, d] and the K pool [pages, nkv, page, d].
//   cache         k and v at `slots` (negative: nothing); V pool [pages, nkv, page, dv] or, grouped, [pages, nkv,
//                 page / 8, dv, 8].
// Sums, norms and the heads' mix are float32; one rounding where a value is stored.
//
// `head_gate_kernel`: x[t, h, :] *= sigmoid(g[t, h]), one number a head (g: columns of a packed projection).
// `rows_rmsnorm_kernel`: rows of a packed projection (a column range) RMS-normed with a weight, float32 inside.
#include "common.h"

namespace xi {

// threads a token: 1024 in steps of few tokens (a row is a few thousand channels: every thread a few, their loads in flight
// at once), 256 where the tokens themselves fill the chip
constexpr int kTapsUnrolled = 8;    // convolutions of up to this many taps ask for all their inputs before the first sum

// four values that follow each other, in one store where the type and the place allow it
__device__ __forceinline__ void store_run4(float* dst, const float (&v)[4]) {
  if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = v[i];
  }
}
__device__ __forceinline__ void store_run4(bf16* dst, const float (&v)[4]) {
  if ((reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
    unsigned u[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const bf16 lo = __float2bfloat16(v[2 * i]), hi = __float2bfloat16(v[2 * i + 1]);
      u[i] = (unsigned)*reinterpret_cast<const unsigned short*>(&lo) | ((unsigned)*reinterpret_cast<const unsigned short*>(&hi) << 16);
    }
    *reinterpret_cast<uint2*>(dst) = make_uint2(u[0], u[1]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = __float2bfloat16(v[i]);
  }
}

template <typename T, int kRowThreads>
__global__ __launch_bounds__(kRowThreads) void conv_qkv_rows_kernel(
    const T* __restrict__ u, long long u_stride, const float* __restrict__ cw, int taps, const float* __restrict__ tails,
    long long tail_stride, const long long* __restrict__ state_slots, const int* __restrict__ tok_seq,
    const int* __restrict__ cu_q, const float* __restrict__ qw, const float* __restrict__ kw, float eps, int v_unit,
    const float* __restrict__ talk, const long long* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int page_size, int nq, int nkv, int d, int dv, int v_grouped) {
  extern __shared__ float row[];                 // the token's C channels after the convolution, then the heads' mix
  __shared__ float scratch[kRowThreads / kWave];
  const int t = blockIdx.x;
  const int nqd = nq * d, nkd = nkv * d, nvd = nkv * dv, C = nqd + nkd + nvd;
  float* talk_s = row + C;                       // [nq, nq]
  if (talk)
    for (int i = threadIdx.x; i < nq * nq; i += kRowThreads) talk_s[i] = talk[i];
  const T* ur = u + (size_t)t * u_stride;
  if (cw && taps <= kTapsUnrolled) {             // four channels a thread at a time, all their inputs asked for before the first sum
    const int b = taps > 1 ? tok_seq[t] : 0;
    const int t0 = taps > 1 ? cu_q[b] : 0;
    const float* tail = taps > 1 ? tails + (size_t)state_slots[b] * tail_stride : nullptr;
    constexpr int kAtOnce = 4;
    for (int c0 = threadIdx.x; c0 < C; c0 += kAtOnce * kRowThreads) {
      float x[kAtOnce][kTapsUnrolled], w[kAtOnce][kTapsUnrolled];
#pragma unroll
      for (int a = 0; a < kAtOnce; ++a) {
        const int c = c0 + a * kRowThreads;
#pragma unroll
        for (int j = 0; j < kTapsUnrolled; ++j) {
          const int s = t - (taps - 1) + j;
          const bool in = j < taps && c < C;
          x[a][j] = !in ? 0.f : s >= t0 ? to_float(u[(size_t)s * u_stride + c]) : tail[(size_t)(taps - 1 - (t0 - s)) * C + c];
          w[a][j] = in ? cw[(size_t)c * taps + j] : 0.f;
        }
      }
#pragma unroll
      for (int a = 0; a < kAtOnce; ++a) {
        const int c = c0 + a * kRowThreads;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < kTapsUnrolled; ++j)
          if (j < taps) acc = fmaf(w[a][j], x[a][j], acc);
        if (c < C) row[c] = acc;
      }
    }
  } else if (cw) {
    const int b = tok_seq[t];
    const int t0 = cu_q[b];
    const float* tail = tails + (size_t)state_slots[b] * tail_stride;
    for (int c = threadIdx.x; c < C; c += kRowThreads) {
      float acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int s = t - (taps - 1) + j;
        // before the portion: s = t0 - k, k = 1 .. taps - 1, the tail's entry taps - 1 - k
        const float x = s >= t0 ? to_float(u[(size_t)s * u_stride + c]) : tail[(size_t)(taps - 1 - (t0 - s)) * C + c];
        acc = fmaf(cw[(size_t)c * taps + j], x, acc);
      }
      row[c] = acc;
    }
  } else {
    for (int c = threadIdx.x; c < C; c += kRowThreads) row[c] = to_float(ur[c]);
  }
  __syncthreads();
  if (qw) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nqd; i += kRowThreads) ss = fmaf(row[i], row[i], ss);
    const float invq = rsqrtf(block_sum<kRowThreads / kWave>(ss, scratch) / (float)nqd + eps);
    ss = 0.f;
    for (int i = threadIdx.x; i < nkd; i += kRowThreads) ss = fmaf(row[nqd + i], row[nqd + i], ss);
    const float invk = rsqrtf(block_sum<kRowThreads / kWave>(ss, scratch) / (float)nkd + eps);
    for (int i = threadIdx.x; i < nqd; i += kRowThreads) row[i] = row[i] * invq * qw[i];
    for (int i = threadIdx.x; i < nkd; i += kRowThreads) row[nqd + i] = row[nqd + i] * invk * kw[i];
  }
  if (v_unit) {                                  // a wave a value head at a time
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int h = wave; h < nkv; h += kRowThreads / kWave) {
      float* vr = row + nqd + nkd + h * dv;
      float ss = 0.f;
      for (int i = lane; i < dv; i += kWave) ss = fmaf(vr[i], vr[i], ss);
      const float inv = rsqrtf(wave_sum(ss) / (float)dv + eps);
      for (int i = lane; i < dv; i += kWave) vr[i] *= inv;
    }
  }
  __syncthreads();
  if (talk && d % 4 == 0 && nq % 4 == 0) {       // four heads by four dims of one kv head a thread: a small product a token,
    const int g = nq / nkv;                      // its operands read from LDS once for sixteen sums
    T* qo = q_out + (size_t)t * nq * nkd;
    const int per_row = nkd / 4;
    for (int i = threadIdx.x; i < (nq / 4) * per_row; i += kRowThreads) {
      const int hb = i / per_row, r = 4 * (i - hb * per_row);
      const int c = r / d, e = r - c * d;
      float acc[4][4] = {};
      for (int j = 0; j < g; ++j) {
        const float4 x = *reinterpret_cast<const float4*>(row + (c * g + j) * d + e);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const float w = talk_s[(4 * hb + a) * nq + c * g + j];
          acc[a][0] = fmaf(w, x.x, acc[a][0]);
          acc[a][1] = fmaf(w, x.y, acc[a][1]);
          acc[a][2] = fmaf(w, x.z, acc[a][2]);
          acc[a][3] = fmaf(w, x.w, acc[a][3]);
        }
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) store_run4(qo + (size_t)(4 * hb + a) * nkd + r, acc[a]);
    }
  } else if (talk) {
    const int g = nq / nkv;
    T* qo = q_out + (size_t)t * nq * nkd;
    for (int i = threadIdx.x; i < nq * nkd; i += kRowThreads) {
      const int h = i / nkd, r = i - h * nkd;
      const int c = r / d, e = r - c * d;
      float acc = 0.f;
      for (int j = 0; j < g; ++j) acc = fmaf(talk_s[h * nq + c * g + j], row[(c * g + j) * d + e], acc);
      qo[i] = from_float<T>(acc);
    }
  } else {
    for (int i = threadIdx.x; i < nqd; i += kRowThreads) q_out[(size_t)t * nqd + i] = from_float<T>(row[i]);
  }
  const long long slot = slots[t];
  if (slot < 0) return;
  const size_t page = (size_t)(slot / page_size);
  const int off = (int)(slot % page_size);
  if (talk) {                                    // one key head of nkv d dims: the row as it is
    T* kr = k_cache + (page * page_size + off) * (size_t)nkd;
    for (int i = threadIdx.x; i < nkd; i += kRowThreads) kr[i] = from_float<T>(row[nqd + i]);
  } else {
    for (int i = threadIdx.x; i < nkd; i += kRowThreads) {
      const int h = i / d, c = i - h * d;
      k_cache[((page * nkv + h) * page_size + off) * d + c] = from_float<T>(row[nqd + i]);
    }
  }
  for (int i = threadIdx.x; i < nvd; i += kRowThreads) {
    const int h = i / dv, c = i - h * dv;
    const size_t base = (page * nkv + h) * (size_t)page_size * dv;
    const size_t at = v_grouped ? base + ((size_t)(off >> 3) * dv + c) * 8 + (off & 7) : base + (size_t)off * dv + c;
    v_cache[at] = from_float<T>(row[nqd + nkd + i]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* __restrict__ x, const T* __restrict__ g, long long g_stride,
                                                        size_t n, int H, int dv) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / ((size_t)H * dv);
  const int h = (int)((i - t * H * dv) / dv);
  const float gv = to_float(g[t * g_stride + h]);
  x[i] = from_float<T>(to_float(x[i]) * (1.f / (1.f + expf(-gv))));
}

// a workgroup a row
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rows_rmsnorm_kernel(const TI* __restrict__ x, long long x_stride,
                                                           const float* __restrict__ w, float eps, TO* __restrict__ out,
                                                           int n_rows, int n) {
  __shared__ float scratch[4];
  const int r = blockIdx.x;
  const TI* xr = x + (size_t)r * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = to_float(xr[i]);
    ss = fmaf(v, v, ss);
  }
  const float inv = rsqrtf(block_sum<4>(ss, scratch) / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += 256) out[(size_t)r * n + i] = from_float<TO>(to_float(xr[i]) * inv * (w ? w[i] : 1.f));
}

}  // namespace xi

using namespace xi;

extern "C" {

// u: rows of u_stride elements in `dtype`, the first C = nq d + nkv d + nkv dv are q, k, v; cw float32 [C, taps] (null:
// no convolution); tails float32, slot s at tails + s * tail_stride, [taps - 1, C]; state_slots int64 [B]; tok_seq int32
// [T]; cu_q int32 [B + 1]; qw, kw float32 or both null; talk float32 [nq, nq] or null; slots int64 [T]; q_out [T, nq,
// nkv d] with talk, else [T, nq, d]; pools as the head of the file says.
int xi_conv_qkv_rows(const void* u, long long u_stride, int dtype, const float* cw, int taps, const float* tails,
                     long long tail_stride, const long long* state_slots, const int* tok_seq, const int* cu_q,
                     const float* qw, const float* kw, float eps, int v_unit, const float* talk, const long long* slots,
                     void* q_out, void* k_cache, void* v_cache, int page_size, int n_tok, int nq, int nkv, int d, int dv,
                     int v_grouped, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && nq > 0 && nkv > 0 && d > 0 && dv > 0 && page_size > 0 && nq % nkv == 0,
           "conv_qkv_rows: bad sizes T=%d nq=%d nkv=%d d=%d dv=%d page=%d", n_tok, nq, nkv, d, dv, page_size);
  const long long C = (long long)nq * d + (long long)nkv * d + (long long)nkv * dv;
  XI_CHECK(u_stride >= C, "conv_qkv_rows: rows of %lld elements do not hold %lld channels", u_stride, C);
  XI_CHECK((qw == nullptr) == (kw == nullptr), "conv_qkv_rows: q and k norm weights must both be given or both absent");
  XI_CHECK(cw == nullptr || taps >= 1, "conv_qkv_rows: a convolution of %d taps", taps);
  XI_CHECK(cw == nullptr || taps == 1 || (tails && state_slots && tok_seq && cu_q && tail_stride >= (taps - 1) * C),
           "conv_qkv_rows: a convolution of %d taps needs the requests' tails", taps);
  XI_CHECK(!v_grouped || page_size % 8 == 0, "conv_qkv_rows: V in groups of eight keys needs pages of a multiple of 8 tokens, not %d",
           page_size);
  const size_t lds = ((size_t)C + (talk ? (size_t)nq * nq : 0)) * sizeof(float);
  XI_CHECK(lds <= 150 * 1024, "conv_qkv_rows: a row of %lld channels (and %d heads' mix) does not fit in LDS", C, nq);
  if (n_tok == 0) return 0;
#define XI_CR(TT)                                                                                                     \
  do {                                                                                                                \
    if (n_tok <= 128) XI_CR_N(TT, 1024);                                                                              \
    else XI_CR_N(TT, 256);                                                                                            \
  } while (0)
#define XI_CR_N(TT, NT)                                                                                               \
  do {                                                                                                                \
    auto kern = conv_qkv_rows_kernel<TT, NT>;                                                                         \
    if (lds > 48 * 1024) {                                                                                            \
      hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);   \
      XI_CHECK(e_ == hipSuccess, "conv_qkv_rows: cannot get %zu bytes of LDS", lds);                                  \
    }                                                                                                                 \
    kern<<<n_tok, NT, lds, stream>>>((const TT*)u, u_stride, cw, taps, tails, tail_stride, state_slots, tok_seq, \
                                              cu_q, qw, kw, eps, v_unit, talk, slots, (TT*)q_out, (TT*)k_cache,       \
                                              (TT*)v_cache, page_size, nq, nkv, d, dv, v_grouped);                    \
  } while (0)
  if (dtype == kF32) XI_CR(float);
  else if (dtype == kBF16) XI_CR(bf16);
  else XI_CHECK(false, "conv_qkv_rows: unknown dtype %d", dtype);
#undef XI_CR
#undef XI_CR_N
  XI_LAUNCH_CHECK("conv_qkv_rows");
  return 0;
}

// x [T, H, dv] in `dtype`, in place; g: rows of g_stride elements whose first H are the heads' gates.
int xi_head_gate(void* x, const void* g, long long g_stride, int dtype, int n_tok, int H, int dv, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && dv > 0 && g_stride >= H, "head_gate: bad sizes T=%d H=%d dv=%d", n_tok, H, dv);
  if (n_tok == 0) return 0;
  const size_t n = (size_t)n_tok * H * dv;
  const size_t blocks = (n + 255) / 256;
  XI_CHECK(blocks < (1ull << 31), "head_gate: too many tokens");
  if (dtype == kF32) head_gate_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((float*)x, (const float*)g, g_stride, n, H, dv);
  else if (dtype == kBF16) head_gate_kernel<bf16><<<(unsigned)blocks, 256, 0, stream>>>((bf16*)x, (const bf16*)g, g_stride, n, H, dv);
  else XI_CHECK(false, "head_gate: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("head_gate");
  return 0;
}

// x: n_rows rows of x_stride elements in `in_dtype`, the first n normed; w float32 [n] or null; out [n_rows, n] in `out_dtype`.
int xi_rows_rmsnorm(const void* x, long long x_stride, int in_dtype, const float* w, float eps, void* out, int out_dtype,
                    int n_rows, int n, hipStream_t stream) {
  XI_CHECK(n_rows >= 0 && n > 0 && x_stride >= n, "rows_rmsnorm: bad sizes rows=%d n=%d", n_rows, n);
  if (n_rows == 0) return 0;
  const unsigned blocks = (unsigned)n_rows;
#define XI_RN(TI, TO) \
  rows_rmsnorm_kernel<TI, TO><<<blocks, 256, 0, stream>>>((const TI*)x, x_stride, w, eps, (TO*)out, n_rows, n)
  if (in_dtype == kF32 && out_dtype == kF32) XI_RN(float, float);
  else if (in_dtype == kF32 && out_dtype == kBF16) XI_RN(float, bf16);
  else if (in_dtype == kBF16 && out_dtype == kBF16) XI_RN(bf16, bf16);
  else if (in_dtype == kBF16 && out_dtype == kF32) XI_RN(bf16, float);
  else XI_CHECK(false, "rows_rmsnorm: unknown dtypes %d, %d", in_dtype, out_dtype);
#undef XI_RN
  XI_LAUNCH_CHECK("rows_rmsnorm");
  return 0;
}

}  // extern "C"
