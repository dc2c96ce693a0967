// Paged causal GQA attention, one workgroup per (token, query head), float32 math.
// It serves every case (prompt portions, decode tokens, windows, any head size) and is
// the attention of the 32-bit path; the bfloat16 path uses it where no faster kernel
// applies.  Keys of a token at position p are the cached positions lo..p of its own
// request, lo = max(0, p - window + 1), read through the request's block table.  K is
// [page, kv_head, offset, d]; V is [page, kv_head, offset, dv] or, with v_grouped,
// [page, kv_head, offset / 8, dv, 8]; the value head size dv may differ from d.
//
// Options of the score, each off unless given:  s = (q . k) * scale;  with a soft cap c,
// s = c * tanh(s / c);  with per-head slopes a[h], s -= a[h] * (p - p') (a bias that grows
// with the distance to the key).  With per-head `sinks` z[h] the softmax's denominator also holds
// exp(z[h]): one more weight, taken as it is, that no value goes with.  With `values_in_keys`
// there is no V pool: a key's first dv dims are its value (attention over a latent).
// The K pool may hold another number of heads than the V pool, `nkk` (query head h reads key head h / (nq / nkk) and
// value head h / (nq / nkv)): one key head of all kv heads' dims side by side serves heads whose scores are mixed.
//
// Reference: PagedAttention::forward at /root/reference/src/models/layers/attention.rs:947-958
// (external kernel); golden formula tests/probes/compare_flashinfer_probe.py:51-73:
//   s[p'] = (q . k[p']) * scale for p' <= p, softmax over them in float32, o = sum a[p'] v[p'];
//   query head h reads kv head h / (nq / nkv).
//
// The order of every reduction is fixed by (position, window) alone: keys are taken in
// chunks of 64 starting at lo, chunk c goes to wave c % 4, and the four partial results
// are merged in wave order.
#include "common.h"

namespace xi {

constexpr int kMaxHeadDim = 256;       // value heads up to this size take the first instantiation,
constexpr int kMaxHeadDimWide = 640;   // up to this the second
constexpr int kMaxKeyDim = 8192;       // key heads: the query sits in LDS, as long as it is
constexpr int kAttnWaves = 4;

template <typename T, int MAXD>
__global__ __launch_bounds__(kAttnWaves* kWave) void attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tok_seq,
    const int* __restrict__ positions, T* __restrict__ out, float scale, int window, int page_size,
    int nq, int nkv, int d, int dv, int v_grouped, float softcap, const float* __restrict__ slopes,
    const float* __restrict__ sinks, int values_in_keys, int nkk) {
  extern __shared__ float q_s[];       // [d]
  __shared__ float acc_s[kAttnWaves][MAXD];
  __shared__ float m_s[kAttnWaves], l_s[kAttnWaves];

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (nq / nkv);
  const int kh = h / (nq / nkk);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int seq = tok_seq[t];
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* bt = block_tables + (size_t)seq * max_pages;

  const T* qp = q + ((size_t)t * nq + h) * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) q_s[i] = to_float(qp[i]);
  __syncthreads();
  const float slope = slopes ? slopes[h] : 0.f;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;

  constexpr int NE = MAXD / kWave;  // output dims per lane
  float acc[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) acc[e] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int n_keys = pos - lo + 1;
  const int n_chunks = (n_keys + kWave - 1) / kWave;
  for (int c = wave; c < n_chunks; c += kAttnWaves) {
    const int key = lo + c * kWave + lane;
    const bool valid = key <= pos;
    int row = 0;  // row of this lane's key in the cache, in units of d elements
    int val = 0;  // and of its value, in units of dv elements
    int vrow = 0, voff = 0;  // grouped V: first row of the (page, kv head) block and the offset
    float s = -INFINITY;
    if (valid) {
      const int page = bt[key / page_size];
      row = (page * nkk + kh) * page_size + key % page_size;
      val = (page * nkv + kvh) * page_size + key % page_size;
      vrow = (page * nkv + kvh) * dv;
      voff = key % page_size;
      const T* kp = k_cache + (size_t)row * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float(kp[i]), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s * inv_cap);
      if (slopes) s -= slope * (float)(pos - key);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // exp(-inf) = 0 on the first chunk
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int e = 0; e < NE; ++e) acc[e] *= corr;
    const int n_in_chunk = min(kWave, pos - (lo + c * kWave) + 1);
    for (int j = 0; j < n_in_chunk; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int rj = __shfl(values_in_keys ? row : val, j, kWave);
      const int vrj = __shfl(vrow, j, kWave);
      const int voj = __shfl(voff, j, kWave);
      const T* vp = values_in_keys ? k_cache + (size_t)rj * d : v_cache + (size_t)rj * dv;
      const T* vtp = v_cache + (size_t)vrj * page_size + (size_t)(voj >> 3) * dv * 8 + (voj & 7);  // [offset / 8, dv, 8] block
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int i = lane + e * kWave;
        if (i < dv) {
          const float vv = v_grouped ? to_float(vtp[(size_t)i * 8]) : to_float(vp[i]);
          acc[e] = fmaf(pj, vv, acc[e]);
        }
      }
    }
  }
  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int i = lane + e * kWave;
    if (i < dv) acc_s[wave][i] = acc[e];
  }
  __syncthreads();
  float mm = m_s[0];
#pragma unroll
  for (int w = 1; w < kAttnWaves; ++w) mm = fmaxf(mm, m_s[w]);
  const float sink = sinks ? sinks[h] : -INFINITY;
  mm = fmaxf(mm, sink);
  float f[kAttnWaves];
  float ll = 0.f;
#pragma unroll
  for (int w = 0; w < kAttnWaves; ++w) {
    f[w] = (m_s[w] == -INFINITY) ? 0.f : expf(m_s[w] - mm);
    ll += l_s[w] * f[w];
  }
  if (sinks) ll += expf(sink - mm);
  T* op = out + ((size_t)t * nq + h) * dv;
  for (int i = threadIdx.x; i < dv; i += blockDim.x) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) o += acc_s[w][i] * f[w];
    op[i] = from_float<T>(o / ll);
  }
}

}  // namespace xi

using namespace xi;

extern "C" int xi_attention_generic(const void* q, const void* k_cache, const void* v_cache,
                                    int dtype, const int* block_tables, int max_pages,
                                    const int* tok_seq, const int* positions, void* out,
                                    float scale, int window, int page_size, int n_tok, int nq,
                                    int nkv, int d, int dv, int v_grouped, float softcap, const float* slopes,
                                    const float* sinks, int values_in_keys, int nkk, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && nq > 0 && nkv > 0 && page_size > 0 && max_pages > 0,
           "attention: bad sizes T=%d nq=%d nkv=%d page=%d max_pages=%d", n_tok, nq, nkv, page_size, max_pages);
  XI_CHECK(nq % nkv == 0, "attention: %d query heads are not a multiple of %d kv heads", nq, nkv);
  XI_CHECK(nkk > 0 && nq % nkk == 0 && (!values_in_keys || nkk == nkv), "attention: %d query heads on %d key heads", nq, nkk);
  XI_CHECK(d > 0 && d <= kMaxKeyDim, "attention: head_dim %d is outside 1..%d", d, kMaxKeyDim);
  XI_CHECK(dv > 0 && dv <= kMaxHeadDimWide, "attention: value head size %d is outside 1..%d", dv, kMaxHeadDimWide);
  XI_CHECK(!values_in_keys || (dv <= d && !v_grouped), "attention: values that are the keys' first dims need dv <= d");
  XI_CHECK(softcap >= 0.f, "attention: the soft cap must be positive (0: none), got %g", (double)softcap);
  XI_CHECK(nq <= 65535, "attention: too many heads (%d)", nq);
  XI_CHECK(!v_grouped || page_size % 8 == 0, "attention: V in groups of eight keys needs pages of a multiple of 8 tokens, not %d", page_size);
  if (n_tok == 0) return 0;
  dim3 grid(n_tok, nq);
  const bool wide = dv > kMaxHeadDim;
  const size_t q_bytes = (size_t)d * sizeof(float);
#define XI_AG(TT, MAXD)                                                                                                 \
  attention_generic_kernel<TT, MAXD><<<grid, kAttnWaves * kWave, q_bytes, stream>>>(                                          \
      (const TT*)q, (const TT*)k_cache, (const TT*)v_cache, block_tables, max_pages, tok_seq, positions, (TT*)out, scale, \
      window, page_size, nq, nkv, d, dv, v_grouped, softcap, slopes, sinks, values_in_keys, nkk)
  if (dtype == kF32 && !wide) XI_AG(float, kMaxHeadDim);
  else if (dtype == kF32) XI_AG(float, kMaxHeadDimWide);
  else if (dtype == kBF16 && !wide) XI_AG(bf16, kMaxHeadDim);
  else if (dtype == kBF16) XI_AG(bf16, kMaxHeadDimWide);
  else XI_CHECK(false, "attention: unknown dtype %d", dtype);
#undef XI_AG
  XI_LAUNCH_CHECK("attention_generic");
  return 0;
}
