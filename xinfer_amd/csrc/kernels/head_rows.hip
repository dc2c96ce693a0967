// A packed projection row [q (nq d) | k (nkv d) | v (nkv dv)] made ready for attention head by head, one wave a
// (token, head):  the first `rot` dims of a q or k head turn by the token's position (pairs (2i, 2i + 1) if
// interleaved, else (i, i + rot / 2); float32 tables [positions, rot / 2]), and then, with `unit`, the head is
// divided by its root mean square over d (eps inside the root; no weight).  q goes to q_out [T, nq, d], k and v
// into the paged cache at `slots` (a negative slot stores nothing).  K pool [pages, nkv, page, d]; V pool
// [pages, nkv, page, dv] or, grouped, [pages, nkv, page / 8, dv, 8].  The value head size may differ from d.
// Everything between the read and the one rounding of the store is float32.
#include "common.h"

namespace xi {

constexpr int kHeadRowWaves = 4;
constexpr int kHeadRowMost = 1024;      // longest head

template <typename T>
__global__ __launch_bounds__(kHeadRowWaves* kWave) void head_rows_kernel(
    const T* __restrict__ qkv, const long long* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int page_size, long long pairs, int nq, int nkv, int d, int dv, int v_grouped,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int interleaved,
    const int* __restrict__ positions, int unit, float eps) {
  extern __shared__ float head_s[];                // [waves][d]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long long pair = (long long)blockIdx.x * kHeadRowWaves + wave;
  if (pair >= pairs) return;
  const int heads = nq + 2 * nkv;
  const long long t = pair / heads;
  const int h = (int)(pair - t * heads);
  const size_t width = (size_t)nq * d + (size_t)nkv * d + (size_t)nkv * dv;
  const T* row = qkv + (size_t)t * width;
  const long long slot = slots[t];
  const size_t page = slot < 0 ? 0 : (size_t)(slot / page_size);
  const int off = slot < 0 ? 0 : (int)(slot % page_size);
  if (h >= nq + nkv) {                             // a value head: a copy
    if (slot < 0) return;
    const int hv = h - nq - nkv;
    const T* src = row + (size_t)(nq + nkv) * d + (size_t)hv * dv;
    const size_t base = (page * nkv + hv) * (size_t)page_size * dv;
    for (int c = lane; c < dv; c += kWave) {
      const size_t at = v_grouped ? base + ((size_t)(off >> 3) * dv + c) * 8 + (off & 7) : base + (size_t)off * dv + c;
      v_cache[at] = src[c];
    }
    return;
  }
  const bool is_q = h < nq;
  if (!is_q && slot < 0) return;
  const T* src = row + (size_t)h * d;              // k heads follow the q heads
  float* x = head_s + (size_t)wave * d;
  const int half = rot / 2;
  const size_t trow = rot ? (size_t)positions[t] * half : 0;
  float ss = 0.f;
  for (int i = lane; i < half; i += kWave) {
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    const float a = to_float(src[ia]), b = to_float(src[ib]);
    const float cs = cos_t[trow + i], sn = sin_t[trow + i];
    const float ra = a * cs - b * sn, rb = b * cs + a * sn;
    x[ia] = ra;
    x[ib] = rb;
    ss = fmaf(ra, ra, fmaf(rb, rb, ss));
  }
  for (int i = rot + lane; i < d; i += kWave) {
    const float a = to_float(src[i]);
    x[i] = a;
    ss = fmaf(a, a, ss);
  }
  const float inv = unit ? rsqrtf(wave_sum(ss) / (float)d + eps) : 1.f;
  __builtin_amdgcn_wave_barrier();
  T* dst = is_q ? q_out + ((size_t)t * nq + h) * d : k_cache + ((page * nkv + (h - nq)) * (size_t)page_size + off) * d;
  // (a lane reads back what it wrote itself: pairs and single dims are dealt out the same way in both loops)
  for (int i = lane; i < half; i += kWave) {
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    dst[ia] = from_float<T>(x[ia] * inv);
    dst[ib] = from_float<T>(x[ib] * inv);
  }
  for (int i = rot + lane; i < d; i += kWave) dst[i] = from_float<T>(x[i] * inv);
}

}  // namespace xi

using namespace xi;

extern "C" int xi_head_rows(const void* qkv, int dtype, const long long* slots, void* q_out, void* k_cache, void* v_cache,
                            int page_size, int n_tok, int nq, int nkv, int d, int dv, int v_grouped, const float* cos_t,
                            const float* sin_t, int rot, int interleaved, const int* positions, int unit, float eps,
                            hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && nq > 0 && nkv > 0 && d > 0 && dv > 0 && page_size > 0,
           "head_rows: bad sizes T=%d nq=%d nkv=%d d=%d dv=%d page=%d", n_tok, nq, nkv, d, dv, page_size);
  XI_CHECK(d <= kHeadRowMost, "head_rows: heads of up to %d dims, not %d", kHeadRowMost, d);
  XI_CHECK(rot >= 0 && rot % 2 == 0 && rot <= d, "head_rows: %d rotated dims of a head of %d", rot, d);
  XI_CHECK(rot == 0 || (cos_t && sin_t && positions), "head_rows: a rotation needs its tables and the positions");
  XI_CHECK(!v_grouped || page_size % 8 == 0, "head_rows: V in groups of eight keys needs pages of a multiple of 8 tokens, not %d",
           page_size);
  if (n_tok == 0) return 0;
  const long long pairs = (long long)n_tok * (nq + 2 * nkv);
  const long long blocks = (pairs + kHeadRowWaves - 1) / kHeadRowWaves;
  XI_CHECK(blocks < (1ll << 31), "head_rows: too many tokens");
  const size_t lds = (size_t)kHeadRowWaves * d * sizeof(float);
  if (dtype == kF32)
    head_rows_kernel<float><<<(unsigned)blocks, kHeadRowWaves * kWave, lds, stream>>>(
        (const float*)qkv, slots, (float*)q_out, (float*)k_cache, (float*)v_cache, page_size, pairs, nq, nkv, d, dv, v_grouped,
        cos_t, sin_t, rot, interleaved, positions, unit, eps);
  else if (dtype == kBF16)
    head_rows_kernel<bf16><<<(unsigned)blocks, kHeadRowWaves * kWave, lds, stream>>>(
        (const bf16*)qkv, slots, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, page_size, pairs, nq, nkv, d, dv, v_grouped, cos_t,
        sin_t, rot, interleaved, positions, unit, eps);
  else
    XI_CHECK(false, "head_rows: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("head_rows");
  return 0;
}
