// An embedding that also looks at the token before, and what a run of layers may add to the stream when
// it starts.
//
// `embed_pair_kernel`: out[t] = float(table[ids[t]]) * scale + float(pairs[row(t)]), the start of the float32
// residual stream.  row(t) = (prev * mul_prev + ids[t] * mul_cur) mod buckets with prev the token before t in
// its sequence, and row `buckets` (the table's last) for a sequence's first token (position 0).  The token
// before the first token of a step's portion is not among the step's tokens: it is what the request's slot of
// `last` holds, which `keep_last_token_kernel` writes after the embedding of every step (a launch of its
// own: the slot is read by the portion's first token and written for its last, which other workgroups hold).
//
// `stream_start_kernel`: x[t] += f * sum_p pending[p][t] (+ first[t]) (+ vec), in that order, all float32: a
// branch that is still to be added, then the embedding's output again, then one row of a table.
#include "common.h"

namespace xi {

template <typename T>
__global__ __launch_bounds__(256) void embed_pair_kernel(const T* __restrict__ table, const T* __restrict__ pairs,
                                                         const int* __restrict__ ids, const int* __restrict__ positions,
                                                         const int* __restrict__ tok_seq, const int* __restrict__ cu_q,
                                                         const long long* __restrict__ slots, const int* __restrict__ last,
                                                         float* __restrict__ out, int H, float scale, long long buckets,
                                                         long long mul_prev, long long mul_cur) {
  const int t = blockIdx.x;
  const int cur = ids[t];
  long long row = buckets;
  if (positions[t] > 0) {
    const int b = tok_seq[t];
    const long long prev = (t == cu_q[b]) ? last[slots[b]] : ids[t - 1];
    row = (prev * mul_prev + (long long)cur * mul_cur) % buckets;
  }
  const T* e = table + (size_t)cur * H;
  const T* p = pairs + (size_t)row * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = fmaf(to_float(e[i]), scale, to_float(p[i]));
}

__global__ void keep_last_token_kernel(const int* __restrict__ ids, const int* __restrict__ cu_q,
                                       const long long* __restrict__ slots, int* __restrict__ last, int n_seqs) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= n_seqs) return;
  const int end = cu_q[b + 1];
  if (end > cu_q[b]) last[slots[b]] = ids[end - 1];
}

template <typename T>
__global__ void stream_start_kernel(float* __restrict__ x, const T* __restrict__ pending, int parts, float factor,
                                    const float* __restrict__ first, const float* __restrict__ vec, int H, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (pending) {
    float s = to_float(pending[i]);
    for (int p = 1; p < parts; ++p) s += to_float(pending[(size_t)p * n + i]);
    v = fmaf(factor, s, v);
  }
  if (first) v += first[i];
  if (vec) v += vec[i % H];
  x[i] = v;
}

}  // namespace xi

using namespace xi;

extern "C" {

// table [V, H] and pairs [buckets + 1, H] in `dtype`; ids, positions, tok_seq int32 [T]; cu_q int32 [B + 1];
// slots int64 [B]; last int32 [slots]; out float32 [T, H].
int xi_embed_pair(const void* table, const void* pairs, int dtype, const int* ids, const int* positions, const int* tok_seq,
                  const int* cu_q, const long long* slots, const int* last, float* out, int n_tok, int H, float scale,
                  long long buckets, long long mul_prev, long long mul_cur, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && buckets > 0, "embed_pair: bad sizes T=%d H=%d buckets=%lld", n_tok, H, buckets);
  XI_CHECK(mul_prev >= 0 && mul_cur >= 0, "embed_pair: the multipliers must not be negative");
  if (n_tok == 0) return 0;
  if (dtype == kF32)
    embed_pair_kernel<float><<<n_tok, 256, 0, stream>>>((const float*)table, (const float*)pairs, ids, positions, tok_seq, cu_q,
                                                        slots, last, out, H, scale, buckets, mul_prev, mul_cur);
  else if (dtype == kBF16)
    embed_pair_kernel<bf16><<<n_tok, 256, 0, stream>>>((const bf16*)table, (const bf16*)pairs, ids, positions, tok_seq, cu_q,
                                                       slots, last, out, H, scale, buckets, mul_prev, mul_cur);
  else
    XI_CHECK(false, "embed_pair: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("embed_pair");
  return 0;
}

int xi_keep_last_token(const int* ids, const int* cu_q, const long long* slots, int* last, int n_seqs, hipStream_t stream) {
  XI_CHECK(n_seqs >= 0, "keep_last_token: bad size %d", n_seqs);
  if (n_seqs == 0) return 0;
  keep_last_token_kernel<<<(n_seqs + 255) / 256, 256, 0, stream>>>(ids, cu_q, slots, last, n_seqs);
  XI_LAUNCH_CHECK("keep_last_token");
  return 0;
}

// x float32 [T, H]; pending null, rows [T, H] in `dtype`, or `parts` float32 partial sums [parts, T, H]; first float32
// [T, H] or null; vec float32 [H] or null.
int xi_stream_start(float* x, const void* pending, int dtype, int parts, float factor, const float* first, const float* vec,
                    int n_tok, int H, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && parts >= 1, "stream_start: bad sizes T=%d H=%d parts=%d", n_tok, H, parts);
  XI_CHECK(parts == 1 || dtype == kF32, "stream_start: partial sums are float32");
  const size_t n = (size_t)n_tok * H;
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == kF32)
    stream_start_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)pending, parts, factor, first, vec, H, n);
  else if (dtype == kBF16)
    stream_start_kernel<bf16><<<blocks, 256, 0, stream>>>(x, (const bf16*)pending, parts, factor, first, vec, H, n);
  else
    XI_CHECK(false, "stream_start: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("stream_start");
  return 0;
}

}  // extern "C"
