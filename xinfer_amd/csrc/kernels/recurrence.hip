// Linear attention with a decaying state (gated linear attention, retention): per request and head a
// matrix S [dk, dv] in float32 that every token updates and reads,
//
//     S <- diag(a_t) S + k_t v_t^T        o_t = S^T q_t
//
// with a_t a decay per key channel.  Two sources of the decay:
//   per head   a_t[i] = decay[h] for every token and channel (retention),
//   per token  a_t[i] = sigmoid(z_t[h, i])^(1 / tau) = exp(-softplus(-z) / tau), z float32 [T, H dk]
//              plus a bias [H dk] (gated linear attention); the logarithm, the exponential and the state
//              are float32;
//   per token and head   a_t[i] = exp(-exp(A[h]) * d_t) for every channel, with the step size d_t = softplus(raw_t[h] +
//              bias[h]) (no clamp) from a column of the projection; the value row is multiplied by d_t as it is read
//              (a selective state space: S <- a_t S + d_t k_t v_t^T).  Step size, exponentials and the product d_t v_t
//              are float32.
//   gates      a_t[i] = gates[t, h, 0] for every channel and the value row times gates[t, h, 1], both made
//              beforehand (float32 [T, H, 2]: the keep and take factors of a matrix memory, mlstm.hip).
// With `v_cols` = dv - 1 the value rows hold v_cols columns a head and the state's last column reads the value 1: it
// is then the sum n of the (decayed, weighted) keys alone, the normalizer of a matrix memory, and its result n . q.
// That column is no lane's: thread c keeps n[c] in a register beside the channel it fetches, and the workgroup adds up
// n[c] q[c] once a token (the grid covers the v_cols columns; the first tile's workgroup writes the column).
// With `group_heads` g > 1, q and k have one set of dk columns for every g heads (head h reads set h / g).
// q, k and v are columns of a packed projection (a row stride and a column offset each); q and k are
// multiplied by `q_scale` / `k_scale` in float32 as they are read.
//
// `linear_scan_kernel`: one workgroup per (item, head, 64 value columns) walks the item's tokens in order,
// from a state it is told to start from, and may leave the new state somewhere.  Lane l owns value column l
// of the tile, wave w the key channels w RPT .. (w + 1) RPT - 1 (read from LDS four at a time; channels past
// the head's are zeros there, so the inner loop has no bounds); a thread keeps its RPT state elements in
// registers for the whole walk.  A token costs one barrier: q, k and the decay of the next token are fetched while this
// one is worked on.  An item is a request's tokens of this step (from the state in its slot, back into it:
// steps of single tokens and short portions; what a token gets then does not depend on how the prompt was
// cut, bit for bit), or one chunk of a long portion:
//
// A long portion is cut into chunks that are walked side by side, in three launches.  (1) every chunk but a
// portion's last, from a zero state and without results: its own share U_c = sum_s (prod_{r > s} a_r) k_s v_s^T
// and the product D_c of its decays; (2) `chunk_carry_kernel`, element by element: the state S_c each chunk
// starts from, S_0 = the slot's, S_{c+1} = D_c S_c + U_c; (3) every chunk from its S_c, with results, the
// portion's last chunk leaving its state in the slot.  Twice the arithmetic of one walk, in a chain a chunk
// long instead of a portion long; all of it float32, so the three launches and the one walk agree to rounding.
//
// `head_norm_gate_kernel`: what follows the state in both mixers: each head's o divided by its root mean
// square over dv (eps inside the root), times a weight [dv] shared by the heads (or none), times silu(g),
// rounded to the activation type for the output projection.
#include "common.h"

namespace xi {

constexpr int kScanWaves = 4;
constexpr int kScanCols = 64;

__device__ __forceinline__ float decay_of(float z, float inv_tau) {
  // sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau); softplus(x) = max(x, 0) + log1p(exp(-|x|))
  const float x = -z;
  const float sp = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
  return expf(-sp * inv_tau);
}

// ONE: a token's decay is one number for all of a head's channels (a constant per head, or from a step size): every
// thread makes it itself and keeps it in a register, and the decays' row in LDS is neither written nor read.
template <typename T, int RPT, bool ONE>
__global__ __launch_bounds__(kScanWaves* kWave) void linear_scan_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau,
    const float* __restrict__ head_decay, const T* __restrict__ step, long long step_stride,
    const float* __restrict__ step_bias, const float* __restrict__ decay_log, const float* __restrict__ gates, int v_cols,
    int group_heads, const float* __restrict__ state_in, long long in_stride, const long long* __restrict__ in_idx,
    float* __restrict__ state_out, long long out_stride, const long long* __restrict__ out_idx,
    const int* __restrict__ first, const int* __restrict__ last, float* __restrict__ out, float* __restrict__ decay_out,
    int H, int dk, int dv, float q_scale, float k_scale) {
  __shared__ __attribute__((aligned(16))) float qs[2][kScanWaves * 64], ks[2][kScanWaves * 64], as[2][kScanWaves * 64];
  __shared__ float part[2][kScanWaves][kScanCols];
  __shared__ float npart[2][kScanWaves];
  const int b = blockIdx.x, h = blockIdx.y, j = blockIdx.z * kScanCols + (threadIdx.x & 63);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t0 = first[b], t1 = last[b];
  if (t1 <= t0) return;
  const bool ones = v_cols < dv;            // the state's last column is the keys' own sum
  const bool col = j < v_cols;
  const long long from = in_idx ? in_idx[b] : -1, to = out_idx ? out_idx[b] : -1;      // negative: from zeros / kept nowhere
  const float* S = state_in + (size_t)(from < 0 ? 0 : from) * in_stride + (size_t)h * dk * dv;
  float s[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = wave * RPT + r;
    s[r] = (from >= 0 && col && i < dk) ? S[(size_t)i * dv + j] : 0.f;
  }
  float all_decays = 1.f;               // of channel c, over the item's tokens
  const int c = threadIdx.x;            // the channel this thread fetches for the workgroup
  float nc = (ones && from >= 0 && c < dk) ? S[(size_t)c * dv + v_cols] : 0.f;
  const float hd = head_decay ? head_decay[h] : 0.f;
  const float zb = (z_bias && c < dk) ? z_bias[h * dk + c] : 0.f;
  const int qk0 = (h / group_heads) * dk;       // the head's set of q and k columns
  const float sb = step ? step_bias[h] : 0.f, rate = step ? -expf(decay_log[h]) : 0.f;
  // the token's step size (1 where the decay has another source): every thread makes its own copy
  auto step_of = [&](int t) {
    if (gates) return gates[((size_t)t * H + h) * 2 + 1];
    if (!step) return 1.f;
    const float x = to_float(step[(size_t)t * step_stride + h]) + sb;
    return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
  };
  auto fetch = [&](int t, float dt, float& fq, float& fk, float& fa) {      // (channels past the head's stay zero)
    if (c < dk) {
      fq = to_float(q[(size_t)t * q_stride + qk0 + c]) * q_scale;
      fk = to_float(k[(size_t)t * k_stride + qk0 + c]) * k_scale;
      if (!ONE) fa = decay_of(z[((size_t)t * H + h) * dk + c] + zb, inv_tau);
    }
    if (ONE) fa = gates ? gates[((size_t)t * H + h) * 2] : step ? expf(rate * dt) : hd;
  };
  float fq = 0.f, fk = 0.f, fa = 0.f;
  float dt = step_of(t0);
  fetch(t0, dt, fq, fk, fa);
  // the token's value is asked for a token ahead as well: no step of the walk waits for memory
  // (a column past the value rows' own reads 1)
  auto value_of = [&](int t) { return j < v_cols ? to_float(v[(size_t)t * v_stride + h * v_cols + j]) : 1.f; };
  float v_next = col ? value_of(t0) * dt : 0.f;
  qs[0][c] = fq;
  ks[0][c] = fk;
  if (!ONE) as[0][c] = fa;
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const int cur = (t - t0) & 1;
    all_decays *= fa;
    const float a_now = fa;
    const float vj = v_next;
    if (ones) {                          // (this token's k and q are in LDS since the last barrier)
      nc = fmaf(a_now, nc, dt * ks[cur][c]);
      const float nq = wave_sum(nc * qs[cur][c]);
      if (out && lane == 0) npart[cur][wave] = nq;
    }
    if (t + 1 < t1) {
      dt = step_of(t + 1);
      fetch(t + 1, dt, fq, fk, fa);
      if (col) v_next = value_of(t + 1) * dt;
    }
    float acc = 0.f;
    const float4* a4 = reinterpret_cast<const float4*>(&as[cur][wave * RPT]);
    const float4* k4 = reinterpret_cast<const float4*>(&ks[cur][wave * RPT]);
    const float4* q4 = reinterpret_cast<const float4*>(&qs[cur][wave * RPT]);
#pragma unroll
    for (int r = 0; r < RPT; r += 4) {
      const float4 av = ONE ? make_float4(a_now, a_now, a_now, a_now) : a4[r / 4];
      const float4 kv = k4[r / 4], qv = q4[r / 4];
      s[r] = fmaf(av.x, s[r], kv.x * vj);
      s[r + 1] = fmaf(av.y, s[r + 1], kv.y * vj);
      s[r + 2] = fmaf(av.z, s[r + 2], kv.z * vj);
      s[r + 3] = fmaf(av.w, s[r + 3], kv.w * vj);
      acc = fmaf(s[r], qv.x, acc);
      acc = fmaf(s[r + 1], qv.y, acc);
      acc = fmaf(s[r + 2], qv.z, acc);
      acc = fmaf(s[r + 3], qv.w, acc);
    }
    if (out) part[cur][wave][lane] = acc;
    if (t + 1 < t1) {
      qs[cur ^ 1][c] = fq;
      ks[cur ^ 1][c] = fk;
      if (!ONE) as[cur ^ 1][c] = fa;
    }
    __syncthreads();
    if (out && wave == 0 && col)
      out[((size_t)t * H + h) * dv + j] = (part[cur][0][lane] + part[cur][1][lane]) + (part[cur][2][lane] + part[cur][3][lane]);
    if (out && ones && blockIdx.z == 0 && threadIdx.x == 0)
      out[((size_t)t * H + h) * dv + v_cols] = (npart[cur][0] + npart[cur][1]) + (npart[cur][2] + npart[cur][3]);
  }
  if (to >= 0) {
    float* D = state_out + (size_t)to * out_stride + (size_t)h * dk * dv;
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
      const int i = wave * RPT + r;
      if (col && i < dk) D[(size_t)i * dv + j] = s[r];
    }
    if (ones && blockIdx.z == 0 && c < dk) D[(size_t)c * dv + v_cols] = nc;
  }
  if (decay_out && blockIdx.z == 0 && c < dk) decay_out[((size_t)b * H + h) * dk + c] = all_decays;
}

// The states that the chunks of long portions start from.  Portion p has n[p] chunks, numbered from c0[p]:
// starts[c0] = the slot's state, starts[c + 1] = decays[c] (per key channel) * starts[c] + shares[c].
// One thread an element of the state, one grid row a portion.
__global__ __launch_bounds__(256) void chunk_carry_kernel(const float* __restrict__ state, long long slot_stride,
                                                          const long long* __restrict__ slots, const int* __restrict__ c0,
                                                          const int* __restrict__ n, const float* __restrict__ shares,
                                                          const float* __restrict__ decays, float* __restrict__ starts,
                                                          int H, int dk, int dv) {
  const int p = blockIdx.y;
  const size_t per = (size_t)H * dk * dv;
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= per) return;
  const size_t hi = e / dv;                 // (head, key channel)
  float s = state[(size_t)slots[p] * slot_stride + e];
  const int first = c0[p], count = n[p];
  for (int c = 0; c < count; ++c) {
    const size_t at = (size_t)(first + c);
    starts[at * per + e] = s;
    if (c + 1 < count) s = fmaf(decays[at * H * dk + hi], s, shares[at * per + e]);
  }
}

// one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             float eps, const T* __restrict__ g, long long g_stride,
                                                             T* __restrict__ out, long long pairs, int H, int dv) {
  const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long long t = pair / H;
  const int h = (int)(pair - t * H);
  const float* x = o + (size_t)pair * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += kWave) ss = fmaf(x[i], x[i], ss);
  const float inv = rsqrtf(wave_sum(ss) / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + (size_t)h * dv;
  T* orow = out + (size_t)pair * dv;
  for (int i = lane; i < dv; i += kWave) {
    const float gv = to_float(gr[i]);
    const float n = x[i] * inv * (w ? w[i] : 1.f);
    orow[i] = from_float<T>(n * (gv / (1.f + expf(-gv))));
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// q, k [T, .] with H dk columns from the given pointers (H / group_heads sets of dk columns if group_heads > 1), v with
// H dv, rows `*_stride` elements apart, in `dtype`; the decay from z float32 [T, H dk] (z_bias float32 [H dk] or null), or
// from head_decay float32 [H], or from step (rows of step_stride elements in `dtype`, H columns: the raw step sizes) with
// step_bias and decay_log float32 [H], or from gates float32 [T, H, 2] (the decay and the factor on the value row): one
// of the four.  v_cols: the columns a head has in v's rows (dv, or fewer: the state's further columns read 1).  Item w walks tokens
// first[w] .. last[w] - 1 from the state state_in + in_idx[w] * in_stride ([H, dk, dv] float32; in_idx null or a
// negative entry: from zeros) and leaves its last state at state_out + out_idx[w] * out_stride (null or negative:
// nowhere); out float32 [T, H, dv] or null (no results); decay_out float32 [items, H, dk] or null: the product of
// each channel's decays over the item.
int xi_linear_scan(const void* q, long long q_stride, const void* k, long long k_stride, const void* v, long long v_stride,
                   int dtype, const float* z, const float* z_bias, float tau, const float* head_decay, const void* step,
                   long long step_stride, const float* step_bias, const float* decay_log, const float* gates, int v_cols,
                   int group_heads, const float* state_in,
                   long long in_stride, const long long* in_idx, float* state_out, long long out_stride,
                   const long long* out_idx, const int* first, const int* last, float* out, float* decay_out, int n_items, int H,
                   int dk, int dv, float q_scale, float k_scale, hipStream_t stream) {
  XI_CHECK(n_items >= 0 && H > 0 && dk > 0 && dv > 0, "linear_scan: bad sizes items=%d H=%d dk=%d dv=%d", n_items, H, dk, dv);
  XI_CHECK(dk <= kScanWaves * 64, "linear_scan: key heads of up to %d channels, not %d", kScanWaves * 64, dk);
  XI_CHECK((z != nullptr) + (head_decay != nullptr) + (step != nullptr) + (gates != nullptr) == 1,
           "linear_scan: a decay per token and channel, per head, per token and head from a step size, or ready-made gates: one of them");
  XI_CHECK(v_cols > 0 && (v_cols == dv || v_cols == dv - 1), "linear_scan: %d value columns in rows for a state of %d", v_cols, dv);
  XI_CHECK(step == nullptr || (step_bias && decay_log && step_stride >= H), "linear_scan: a step size needs its bias and its rate");
  XI_CHECK(group_heads >= 1 && H % group_heads == 0, "linear_scan: %d heads in groups of %d", H, group_heads);
  XI_CHECK(z == nullptr || tau > 0.f, "linear_scan: tau must be positive");
  XI_CHECK((in_idx == nullptr || (state_in && in_stride >= (long long)H * dk * dv)) &&
               (out_idx == nullptr || (state_out && out_stride >= (long long)H * dk * dv)),
           "linear_scan: states need a place of at least H dk dv floats each");
  XI_CHECK(first && last, "linear_scan: the items' token ranges are missing");
  if (n_items == 0) return 0;
  dim3 grid((unsigned)n_items, (unsigned)H, (unsigned)((v_cols + kScanCols - 1) / kScanCols));
  XI_CHECK(grid.y <= 65535u && grid.z <= 65535u, "linear_scan: too many heads or value columns");
  const float inv_tau = z ? 1.f / tau : 0.f;
  const int rpt = (dk + kScanWaves - 1) / kScanWaves;
#define XI_SCAN_ARGS(TT)                                                                                                      \
      (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v, v_stride, z, z_bias, inv_tau, head_decay, (const TT*)step,    \
      step_stride, step_bias, decay_log, gates, v_cols, group_heads, state_in, in_stride,                                                    \
      in_idx, state_out, out_stride, out_idx, first, last, out, decay_out, H, dk, dv, q_scale, k_scale
#define XI_SCAN(TT, R)                                                                                                        \
  do {                                                                                                                        \
    if (z) linear_scan_kernel<TT, R, false><<<grid, kScanWaves * kWave, 0, stream>>>(XI_SCAN_ARGS(TT));                       \
    else linear_scan_kernel<TT, R, true><<<grid, kScanWaves * kWave, 0, stream>>>(XI_SCAN_ARGS(TT));                          \
  } while (0)
#define XI_SCAN_T(TT)            \
  do {                           \
    if (rpt <= 8) XI_SCAN(TT, 8); \
    else if (rpt <= 16) XI_SCAN(TT, 16); \
    else if (rpt <= 32) XI_SCAN(TT, 32); \
    else XI_SCAN(TT, 64);        \
  } while (0)
  if (dtype == kF32) XI_SCAN_T(float);
  else if (dtype == kBF16) XI_SCAN_T(bf16);
  else XI_CHECK(false, "linear_scan: unknown dtype %d", dtype);
#undef XI_SCAN_T
#undef XI_SCAN
#undef XI_SCAN_ARGS
  XI_LAUNCH_CHECK("linear_scan");
  return 0;
}

// state float32, slot s at state + s * slot_stride; slots int64 [P]; c0, n int32 [P]; shares, starts float32
// [chunks, H, dk, dv]; decays float32 [chunks, H, dk].
int xi_chunk_carry(const float* state, long long slot_stride, const long long* slots, const int* c0, const int* n,
                   const float* shares, const float* decays, float* starts, int n_portions, int H, int dk, int dv,
                   hipStream_t stream) {
  XI_CHECK(n_portions >= 0 && H > 0 && dk > 0 && dv > 0, "chunk_carry: bad sizes portions=%d H=%d dk=%d dv=%d", n_portions, H, dk, dv);
  XI_CHECK(slot_stride >= (long long)H * dk * dv, "chunk_carry: a state slot is too small");
  if (n_portions == 0) return 0;
  const size_t per = (size_t)H * dk * dv;
  dim3 grid((unsigned)((per + 255) / 256), (unsigned)n_portions);
  XI_CHECK(grid.y <= 65535u, "chunk_carry: too many portions");
  chunk_carry_kernel<<<grid, 256, 0, stream>>>(state, slot_stride, slots, c0, n, shares, decays, starts, H, dk, dv);
  XI_LAUNCH_CHECK("chunk_carry");
  return 0;
}

// o float32 [T, H, dv]; w float32 [dv] or null; g rows of g_stride elements holding [H dv] gates in `dtype`;
// out [T, H dv] in `dtype`.
int xi_head_norm_gate(const float* o, const float* w, float eps, const void* g, long long g_stride, void* out, int dtype,
                      int n_tok, int H, int dv, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && dv > 0 && g_stride >= (long long)H * dv, "head_norm_gate: bad sizes T=%d H=%d dv=%d", n_tok, H,
           dv);
  if (n_tok == 0) return 0;
  const long long pairs = (long long)n_tok * H;
  const long long blocks = (pairs + 3) / 4;
  XI_CHECK(blocks < (1ll << 31), "head_norm_gate: too many tokens");
  if (dtype == kF32)
    head_norm_gate_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(o, w, eps, (const float*)g, g_stride, (float*)out, pairs,
                                                                       H, dv);
  else if (dtype == kBF16)
    head_norm_gate_kernel<bf16><<<(unsigned)blocks, 256, 0, stream>>>(o, w, eps, (const bf16*)g, g_stride, (bf16*)out, pairs, H,
                                                                      dv);
  else
    XI_CHECK(false, "head_norm_gate: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

}  // extern "C"
