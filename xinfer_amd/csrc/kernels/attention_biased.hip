// bfloat16 paged causal GQA attention on the gfx950 matrix cores for scores with options and for
// values of their own head size: the kernel of attention_prefill.hip (K and V^T tiles of 64 keys
// staged through LDS, S^T = K . Q^T, softmax state in the query's lanes, P^T fed to the second
// product from registers) with
//   - the key head size d (K steps of 32: KC) and the value head size dv (row tiles of 16: DT)
//     chosen apart, the V pool being [page, kv_head, offset / 8, dv, 8];
//   - the score made in float32 before the softmax: t = (q . k) * scale; with a soft cap c,
//     t = c * tanh(t / c); with a slope a[h] of the head, t -= a[h] * (i - j) for query position i
//     and key position j; then the mask (causal, window).  tanh(x) = 1 - 2 / (2^(2 x log2 e) + 1):
//     one exponential and one reciprocal a score beside the softmax's own exponential, which is
//     why this kernel spends more of its time outside the matrix cores than the plain one.
//   - a K pool of fewer heads than the V pool (`nkk`, a divisor of nkv: kv head c reads key head c / (nkv / nkk));
//     one key head of all kv heads' dims side by side serves heads whose scores are mixed.
// It serves every mix of prompt portions and single tokens (a single token is a block of one
// query position); the host lays out `tiles` as for the plain kernel.
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float kLog2eB = 1.4426950408889634f;
constexpr int kKeysB = 64;    // keys per tile (two steps of 32)
constexpr int kVPadB = 8;     // bf16 elements of padding per LDS row
constexpr float kSlackB = 8.f;  // how far (log2) a score may exceed the softmax reference point

static __device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
static __device__ __forceinline__ void st8(bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
static __device__ __forceinline__ bf16x8 zero8p() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// NWV waves of NQT column tiles each: the workgroup's NWV * NQT tiles are (position block,
// head) pairs, GH heads per position block.  Eight waves of two tiles keep a wave within
// half of a SIMD's registers, so two waves share a SIMD and one's exponentials overlap the
// other's matrix instructions.
// FULLD: head_dim is exactly 16 * DT, so no row tile of V^T lies past the end and the
// products with V^T are straight-line code.
template <int KC, int DT, int NQT, int GH, int NWV, bool FULLD>
__global__ __launch_bounds__(64 * NWV, 2) void attn_biased_lds_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ vt_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tiles,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, bf16* __restrict__ out, float scale,
    float softcap, const float* __restrict__ slopes, const float* __restrict__ sinks, int window, int page_shift, int nq,
    int nkv, int d, int dv, float* __restrict__ part_o, float* __restrict__ part_ml, int split_keys, int max_splits,
    int rows_heads, int nkk, int rows_kv) {
  const int page = 1 << page_shift;
  constexpr int NT = 64 * NWV;                    // threads
  constexpr int QB = 16 * (NWV * NQT / GH);       // query positions per workgroup
  constexpr int LI = (256 * KC + NT - 1) / NT;    // 16-byte chunks per thread and tile of K
  constexpr int LV = (128 * DT + NT - 1) / NT;    // and of V^T (dv rows of 8 key groups, dv <= 16 DT)
  static_assert((NWV * NQT) % GH == 0, "tiles must divide into whole position blocks");
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int krow = 32 * KC + kVPadB;  // elements per K row in LDS: head_dim rounded up to the
                                         // 32-wide steps of the matrix product (the rest is zero)
  const int vrow = kKeysB + kVPadB;       // elements per V^T row in LDS
  const int stage = kKeysB * krow + dv * vrow;
  bf16* lds = reinterpret_cast<bf16*>(smem);
  int* bt_s = reinterpret_cast<int*>(smem + 2 * (size_t)stage * sizeof(bf16));  // [max_pages]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int g = nq / nkv, groups = g / GH;
  const int kvh = blockIdx.x / groups;
  const int h0 = kvh * g + (blockIdx.x - kvh * groups) * GH;
  const int kh = kvh / (nkv / nkk);               // the kv head's key head
  const int seq = tiles[2 * blockIdx.y], q0_blk = tiles[2 * blockIdx.y + 1];
  const int q_begin = cu_q[seq], q_rows = cu_q[seq + 1] - q_begin;
  const int ctx = ctx_lens[seq];
  // rows_heads with rows_kv > 1: the rows are heads that share the one key head and read rows_kv value heads, rows_heads
  // / rows_kv rows each; a block's rows lie within one value head's rows (the host cuts the blocks so)
  int v_heads = nkv, v_head = kvh, q_len = q_rows;
  if (rows_heads > 0 && rows_kv > 1) {
    const int per = rows_heads / rows_kv;
    v_heads = rows_kv;
    v_head = q0_blk / per;
    q_len = min(q_rows, (v_head + 1) * per);
  }
  // rows_heads > 0: the sequence's rows are the query heads of its one new token (all of them read the one kv head:
  // attention over a latent), so every row stands at the last position and row i has sink i
  const int step = rows_heads > 0 ? 0 : 1;
  const int pos0 = rows_heads > 0 ? ctx - 1 : ctx - q_len;         // position of the portion's first token
  const int k_last = ctx - 1;
  {
    const int* bt = block_tables + (size_t)seq * max_pages;
    const int n_pages = (k_last + page) / page;    // pages that hold keys 0..k_last
    for (int i = threadIdx.x; i < n_pages; i += NT) bt_s[i] = bt[i];
  }

  // keys the workgroup walks
  const int wg_nq = min(QB, q_len - q0_blk);
  const int wg_first = pos0 + step * q0_blk, wg_last = wg_first + step * (wg_nq - 1);
  const int wg_lo = (window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0;
  const int k_begin = wg_lo & ~(kKeysB - 1);
  // split_keys > 0 (steps of single tokens): this workgroup walks one slice of the keys, slice
  // blockIdx.z of `split_keys` keys, and leaves its sums unnormalized for the combine kernel
  const int kt_begin = k_begin + (split_keys > 0 ? (int)blockIdx.z * split_keys : 0);
  const int kt_end = split_keys > 0 ? min(wg_last, kt_begin + split_keys - 1) : wg_last;
  if (split_keys > 0 && kt_begin > wg_last) {          // a slice past the sequence's keys: it says so and ends
    if (rows_heads > 0) {                              // every row of the block (nq is 1)
      for (int i = threadIdx.x; i < wg_nq; i += NT) {
        float* ml = part_ml + (((size_t)(q_begin + q0_blk + i) * nq + h0) * max_splits + blockIdx.z) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
      return;
    }
    for (int ct = 0; ct < NQT; ++ct) {
      const int tile = (threadIdx.x >> 6) * NQT + ct;
      if (tile < GH && (threadIdx.x & 63) == 0) {
        float* ml = part_ml + (((size_t)q_begin * nq + h0 + tile) * max_splits + blockIdx.z) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
    }
    return;
  }

  // this wave's queries: the position blocks its tiles lie in
  const int pb_lo = (wave * NQT) / GH, pb_hi = (wave * NQT + NQT - 1) / GH;
  const int q0 = q0_blk + 16 * pb_lo;
  const bool active = q0 < q_len;
  const int n_q = active ? min(16 * (pb_hi - pb_lo + 1), q_len - q0) : 0;
  const int first_pos = pos0 + step * q0, last_pos = first_pos + step * (n_q - 1);
  const int lo_first = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int lo_last = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int wave_k_begin = lo_first & ~31;

  bf16x8 qb[NQT][KC];
  f32x4 acc[DT][NQT];
  float m_run[NQT], l_run[NQT];
  int qpos[NQT], qlo[NQT];
  float slope2[NQT];                   // the head's slope in the exponent's unit (times log2 e)
#pragma unroll
  for (int ct = 0; ct < NQT; ++ct) {
    const int tile = wave * NQT + ct;
    const int pb = tile / GH, hh = tile - pb * GH;
    slope2[ct] = slopes ? slopes[h0 + hh] * kLog2eB : 0.f;
    const int qi = q0_blk + 16 * pb + r;
    const bool ok = active && qi < q_len;
    qpos[ct] = ok ? pos0 + step * qi : -1;
    qlo[ct] = (ok && window > 0 && qpos[ct] - window + 1 > 0) ? qpos[ct] - window + 1 : 0;
    const bf16* qrow = q + ((size_t)(q_begin + (ok ? qi : 0)) * nq + h0 + hh) * d;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int off = 32 * c + 8 * j;
      qb[ct][c] = (ok && off < d) ? ld8(qrow + off) : zero8p();
    }
    m_run[ct] = -INFINITY;
    l_run[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- cooperative tile copy.  K tile: 64 keys of 4*KC 16-byte chunks (chunks past
  // head_dim are zero), thread t moves chunks t, t + 256, ...; in LDS the keys of each
  // 32-key step are permuted so that the 16 rows one matrix operand reads are consecutive:
  // key k sits at row 16*((k>>2)&1) + 4*(k>>3) + (k&3) of its step.  V^T tile: d rows of 8
  // key groups; thread t moves row t % d of key group t / d, .. (the pool keeps a key group's rows
  // side by side: threads that follow each other read 16 bytes that follow each other).
  constexpr int CPK = 4 * KC;        // chunks per K row in LDS
  const int n_vchunks = 8 * dv;
  int c_kl[LI], c_koff[LI], c_kdst[LI], c_vdst[LV], c_vrow[LV], c_vkg[LV];
#pragma unroll
  for (int i = 0; i < LI; ++i) {
    const int idx = tid + NT * i;
    const int kl = (idx / CPK) & 63, ch = idx % CPK;     // (a thread past the tile's 64 keys repeats one of them)
    const int k32 = kl & 31;
    c_kl[i] = kl;
    c_koff[i] = 8 * ch < d ? 8 * ch : -1;       // -1: a chunk of zeros
    c_kdst[i] = ((kl & 32) + 16 * ((k32 >> 2) & 1) + 4 * (k32 >> 3) + (k32 & 3)) * krow + 8 * ch;
  }
#pragma unroll
  for (int i = 0; i < LV; ++i) {
    const int idx = tid + NT * i;
    c_vkg[i] = idx / dv;
    c_vrow[i] = idx - c_vkg[i] * dv;
    if (c_vkg[i] > 7) { c_vkg[i] = 7; c_vrow[i] = dv - 1; }      // past the tile: read again what the last chunk reads, store nothing
    c_vdst[i] = c_vrow[i] * vrow + 8 * c_vkg[i];
  }
  const size_t k_head_stride = (size_t)d << page_shift;      // elements of one (page, kv head) block of K
  const size_t v_head_stride = (size_t)dv << page_shift;     // and of V
  bf16x8 kreg[LI], vreg[LV];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < LI; ++i) {
      int key = kb + c_kl[i];
      key = key > k_last ? k_last : key;
      const int kp = bt_s[key >> page_shift];
      const bf16* ksrc = k_cache + ((size_t)kp * nkk + kh) * k_head_stride +
                         (size_t)(key & (page - 1)) * d + (c_koff[i] < 0 ? 0 : c_koff[i]);
      kreg[i] = ld8(ksrc);
    }
#pragma unroll
    for (int i = 0; i < LV; ++i) {
      int key0 = kb + 8 * c_vkg[i];
      key0 = key0 > k_last ? (k_last & ~7) : key0;
      const int vp = bt_s[key0 >> page_shift];
      vreg[i] = ld8(vt_cache + ((size_t)vp * v_heads + v_head) * v_head_stride +
                    ((size_t)((key0 & (page - 1)) >> 3) * dv + c_vrow[i]) * 8);     // [offset / 8, dv, 8]
    }
  };
  auto stash = [&](int buf) {
    bf16* Ks = lds + buf * stage;
    bf16* Vs = Ks + kKeysB * krow;
#pragma unroll
    for (int i = 0; i < LI; ++i)
      if (tid + NT * i < 64 * CPK) st8(Ks + c_kdst[i], c_koff[i] < 0 ? zero8p() : kreg[i]);
#pragma unroll
    for (int i = 0; i < LV; ++i)
      if (tid + NT * i < n_vchunks) st8(Vs + c_vdst[i], vreg[i]);
  };

  const float cap2 = softcap > 0.f ? 2.f * kLog2eB / softcap : 0.f;
  __syncthreads();   // the block table is in LDS
  fetch(kt_begin);
  stash(0);
  // every load so far (the queries among them) has landed before the loop starts, so that
  // inside it only the tile in flight is ever waited for: vmcnt(0), other counters untouched
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  int buf = 0;
  for (int kt = kt_begin; kt <= kt_end; kt += kKeysB) {
    const bool more = kt + kKeysB <= kt_end;
    if (more) fetch(kt + kKeysB);
#pragma unroll
    for (int sub = 0; sub < kKeysB / 32; ++sub) {
    const int kb = kt + 32 * sub;
    if (active && kb >= wave_k_begin && kb <= last_pos) {
      const bf16* Ks = lds + buf * stage + 32 * sub * krow;
      const bf16* Vs = lds + buf * stage + kKeysB * krow + 32 * sub;
      // a step needs the mask unless every key is at or before every query and inside every window
      const bool masked = (kb + 31 > first_pos) || (kb < lo_last);
      bf16x8 ka[2][KC];
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const int off = 32 * c + 8 * j;
        ka[0][c] = ld8(Ks + r * krow + off);
        ka[1][c] = ld8(Ks + (16 + r) * krow + off);
      }
      // ---- all scores of the step first: 2 * KC * NQT matrix instructions with nothing
      // between them that waits for their results
      f32x4 s0[NQT], s1[NQT];
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        s0[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        s1[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int c = 0; c < KC; ++c)
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct) {
          s0[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[0][c], qb[ct][c], s0[ct], 0, 0, 0);
          s1[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[1][c], qb[ct][c], s1[ct], 0, 0, 0);
        }
      // ---- the score itself, in the exponent's unit: scale, soft cap, distance bias; then the mask
      {
        const int key0 = kb + 8 * j;
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct) {
          const float dist0 = (float)(qpos[ct] - key0);
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float t0 = s0[ct][v] * scale, t1 = s1[ct][v] * scale;
            if (softcap > 0.f) {
              // c tanh(t / c) = c - 2 c / (2^(2 t log2e / c) + 1); cap2 = 2 log2e / c
              const float e0 = __builtin_amdgcn_exp2f(t0 * cap2), e1 = __builtin_amdgcn_exp2f(t1 * cap2);
              t0 = softcap - 2.f * softcap * __builtin_amdgcn_rcpf(e0 + 1.f);
              t1 = softcap - 2.f * softcap * __builtin_amdgcn_rcpf(e1 + 1.f);
            }
            s0[ct][v] = fmaf(t0, kLog2eB, -slope2[ct] * (dist0 - (float)v));
            s1[ct][v] = fmaf(t1, kLog2eB, -slope2[ct] * (dist0 - (float)(4 + v)));
          }
        }
        if (masked) {
#pragma unroll
          for (int ct = 0; ct < NQT; ++ct)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              if (key0 + v > qpos[ct] || key0 + v < qlo[ct]) s0[ct][v] = -INFINITY;
              if (key0 + 4 + v > qpos[ct] || key0 + 4 + v < qlo[ct]) s1[ct][v] = -INFINITY;
            }
        }
      }
      // ---- this lane's largest score per column tile (raw: the scale is positive and is
      // applied with the shift).  The reference point m_run of the exponentials only has to
      // be near the maximum: it moves when some score exceeds it by more than 2^kSlackB, which
      // is rare after the first keys; then the sums so far are rescaled.  P stays below
      // 2^kSlackB.  One test for all column tiles keeps the common path free of branches.
      float mx[NQT];
      bool moved = false;
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        mx[ct] = fmaxf(fmaxf(fmaxf(s0[ct][0], s0[ct][1]), fmaxf(s0[ct][2], s0[ct][3])),
                       fmaxf(fmaxf(s1[ct][0], s1[ct][1]), fmaxf(s1[ct][2], s1[ct][3])));
        moved = moved || (mx[ct] > m_run[ct] + kSlackB);
      }
      if (__any(moved)) {
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct) {
          float mc = mx[ct];
          mc = fmaxf(mc, lane_xor<16>(mc));
          mc = fmaxf(mc, lane_xor<32>(mc));
          const float m_new = fmaxf(m_run[ct], mc);
          const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[ct] - m_new);
          l_run[ct] *= corr;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            acc[dt][ct][0] *= corr;
            acc[dt][ct][1] *= corr;
            acc[dt][ct][2] *= corr;
            acc[dt][ct][3] *= corr;
          }
          m_run[ct] = m_new;
        }
      }
      // ---- exponentials, then the products with V^T: straight-line code
      bf16x8 pb_[NQT];
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        const float m_safe = (m_run[ct] == -INFINITY) ? 0.f : m_run[ct];
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float p0 = __builtin_amdgcn_exp2f(s0[ct][v] - m_safe);
          const float p1 = __builtin_amdgcn_exp2f(s1[ct][v] - m_safe);
          psum += p0 + p1;
          pb_[ct][v] = (__bf16)p0;
          pb_[ct][4 + v] = (__bf16)p1;
        }
        l_run[ct] += psum;
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        if (FULLD || 16 * dt < dv) {
          const bf16x8 va = ld8(Vs + (16 * dt + r) * vrow + 8 * j);
#pragma unroll
          for (int ct = 0; ct < NQT; ++ct)
            acc[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb_[ct], acc[dt][ct], 0, 0, 0);
        }
      }
    }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  if (!active) return;
#pragma unroll
  for (int ct = 0; ct < NQT; ++ct) {
    float lt = l_run[ct] + lane_xor<16>(l_run[ct]);
    lt += lane_xor<32>(lt);
    const int tile = wave * NQT + ct;
    const int pb = tile / GH, hh = tile - pb * GH;
    const int qi = q0_blk + 16 * pb + r;
    if (qi >= q_len) continue;
    if (split_keys > 0) {
      const size_t at = ((size_t)(q_begin + qi) * nq + h0 + hh) * max_splits + blockIdx.z;
      if (j == 0) {
        part_ml[at * 2] = m_run[ct];
        part_ml[at * 2 + 1] = lt;
      }
      float* po = part_o + at * dv;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        if (16 * dt + 4 * j >= dv) break;
        *reinterpret_cast<f32x4*>(po + 16 * dt + 4 * j) = acc[dt][ct];
      }
      continue;
    }
    // a sink: one more weight in the denominator, exp(sink) on the scale of the reference point, with no value
    if (sinks) lt += __builtin_amdgcn_exp2f(sinks[rows_heads > 0 ? qi : h0 + hh] * kLog2eB - m_run[ct]);
    const float inv = 1.f / lt;
    bf16* o = out + ((size_t)(q_begin + qi) * nq + h0 + hh) * dv;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt + 4 * j >= dv) break;      // dv is a multiple of 8: a lane's four dims lie inside or outside together
      bf16* op = o + 16 * dt + 4 * j;
      const f32x4 a = acc[dt][ct];
      op[0] = __float2bfloat16(a[0] * inv);
      op[1] = __float2bfloat16(a[1] * inv);
      op[2] = __float2bfloat16(a[2] * inv);
      op[3] = __float2bfloat16(a[3] * inv);
    }
  }
}

// Sums of the slices of a token's keys put together: out = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M), in slice
// order (m_s: the slice's reference point in the exponent's unit; a slice without keys has m_s = -inf).
__global__ __launch_bounds__(64) void attn_biased_combine_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml, bf16* __restrict__ out,
                                                                 const float* __restrict__ sinks, int max_splits, int nq,
                                                                 int dv, int rows_heads) {
  const int head = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
  // the head's sink in the exponent's unit (rows_heads > 0: row t is head t % rows_heads of its token)
  const float sink2 = sinks ? sinks[rows_heads > 0 ? t % rows_heads : head] * kLog2eB : -INFINITY;
  const size_t base = ((size_t)t * nq + head) * max_splits;
  __shared__ float f_s[64];
  if (max_splits <= 64) {          // a slice a lane: one round of loads for the weights, one for the sums
    float ms = -INFINITY, ls = 0.f;
    if (lane < max_splits) {
      const float2 ml = *reinterpret_cast<const float2*>(part_ml + (base + lane) * 2);
      ms = ml.x;
      ls = ml.y;
    }
    const float mm = wave_max(ms);
    const float f = ms > -INFINITY ? __builtin_amdgcn_exp2f(ms - mm) : 0.f;
    const float inv = 1.f / (wave_sum(ls * f) + (sinks ? __builtin_amdgcn_exp2f(sink2 - mm) : 0.f));
    f_s[lane] = f;
    __syncthreads();
    for (int i = lane; i < dv; i += 64) {
      float o = 0.f;
      // every slice's sum is asked for, eight at a time (a slice without keys left its place unwritten: what is read
      // there is not used)
#pragma unroll 8
      for (int s2 = 0; s2 < max_splits; ++s2) {
        const float fs = f_s[s2];
        const float v = part_o[(base + s2) * dv + i];
        o += fs > 0.f ? v * fs : 0.f;
      }
      out[((size_t)t * nq + head) * dv + i] = __float2bfloat16(o * inv);
    }
    return;
  }
  float mm = -INFINITY;
  for (int s2 = 0; s2 < max_splits; ++s2) mm = fmaxf(mm, part_ml[(base + s2) * 2]);
  float ll = 0.f;
  for (int s2 = 0; s2 < max_splits; ++s2) {
    const float ms = part_ml[(base + s2) * 2];
    if (ms > -INFINITY) ll += part_ml[(base + s2) * 2 + 1] * __builtin_amdgcn_exp2f(ms - mm);
  }
  if (sinks) ll += __builtin_amdgcn_exp2f(sink2 - mm);
  const float inv = 1.f / ll;
  for (int i = lane; i < dv; i += 64) {
    float o = 0.f;
    for (int s2 = 0; s2 < max_splits; ++s2) {
      const float ms = part_ml[(base + s2) * 2];
      if (ms > -INFINITY) o += part_o[(base + s2) * dv + i] * __builtin_amdgcn_exp2f(ms - mm);
    }
    out[((size_t)t * nq + head) * dv + i] = __float2bfloat16(o * inv);
  }
}

// Column tiles of a workgroup by the larger of the two head sizes and the shape (as the plain kernel:
// eight waves of two tiles up to 128, of one tile above; the small shape has four waves).
static inline int tiles_of_b(int dmax, int small) { return (dmax <= 128 ? 16 : 8) / (small ? 2 : 1); }
static inline int heads_together_b(int g) { return g % 4 == 0 ? 4 : (g % 2 == 0 ? 2 : 1); }

}  // namespace xi

using namespace xi;

extern "C" {

// Sizes the kernel takes: head sizes that are multiples of 8 up to 256, pages a power of two of at least 8.
int xi_attention_biased_supported(int nq, int nkv, int d, int dv, int page) {
  if (nq <= 0 || nkv <= 0 || nq % nkv) return 0;
  if (d <= 0 || d > 256 || d % 8 || dv <= 0 || dv > 256 || dv % 8) return 0;
  if (page < 8 || (page & (page - 1))) return 0;
  return 1;
}

// Query positions per workgroup (the host builds `tiles` in steps of it).
int xi_attention_biased_block(int d, int dv, int g, int small) {
  return 16 * (tiles_of_b(d > dv ? d : dv, small) / heads_together_b(g));
}

// tiles int32 [n_tiles, 2] = (sequence, first query position of the block within the sequence's portion).
// q [T, nq, d]; K pool [pages, nkv, page, d]; V pool [pages, nkv, page / 8, dv, 8]; out [T, nq * dv].
// rows_heads H > 0 (nq = nkv = 1): the rows of a sequence are the H heads of its one token; rows_kv G > 1: the V pool has
// G heads, rows h H / G .. (h + 1) H / G - 1 read value head h, and no block of `tiles` crosses such a border.
// softcap 0: none; slopes null: none; sinks null: none, else float32 [nq], exp(sinks[h]) joins head h's denominator.
int xi_attention_biased_bf16(const void* q, const void* k_cache, const void* vt_cache, const int* block_tables,
                             int max_pages, const int* tiles, int n_tiles, const int* cu_q, const int* ctx_lens,
                             void* out, float scale, float softcap, const float* slopes, const float* sinks, int window,
                             int page, int nq, int nkv, int d, int dv, int small, float* part_o, float* part_ml, int split_keys,
                             int max_splits, int n_tok, int rows_heads, int nkk, int rows_kv, hipStream_t stream) {
  XI_CHECK(rows_kv >= 1 && (rows_kv == 1 || (rows_heads > 0 && rows_heads % rows_kv == 0)),
           "attention_biased: %d value heads for rows that are %d heads", rows_kv, rows_heads);
  XI_CHECK(nkk > 0 && nkv % nkk == 0, "attention_biased: %d kv heads on %d key heads", nkv, nkk);
  XI_CHECK(rows_heads == 0 || (rows_heads > 0 && nq == 1 && nkv == 1 && slopes == nullptr && n_tok % rows_heads == 0),
           "attention_biased: rows that are the %d heads of a token come with one head, no slopes and whole tokens", rows_heads);
  XI_CHECK(xi_attention_biased_supported(nq, nkv, d, dv, page), "attention_biased: unsupported sizes nq=%d nkv=%d d=%d dv=%d page=%d",
           nq, nkv, d, dv, page);
  XI_CHECK(n_tiles >= 0 && n_tiles <= 65535, "attention_biased: %d query blocks are too many for one launch", n_tiles);
  XI_CHECK(softcap >= 0.f, "attention_biased: the soft cap must be positive (0: none)");
  // slices of the keys: for steps in which every sequence brings one token (a tile a token), partial sums
  // part_o float32 [n_tok, nq, max_splits, dv] and part_ml [n_tok, nq, max_splits, 2] from the caller
  XI_CHECK(split_keys == 0 || (split_keys > 0 && split_keys % kKeysB == 0 && max_splits > 0 && max_splits <= 65535 &&
                               part_o != nullptr && part_ml != nullptr && (n_tiles == n_tok || rows_heads > 0) && dv % 4 == 0),
           "attention_biased: slices of %d keys (%d of them) need steps of single tokens and room for the partial sums",
           split_keys, max_splits);
  if (n_tiles == 0) return 0;
  const int g = nq / nkv;
  const int gh = heads_together_b(g);
  dim3 grid(nkv * (g / gh), n_tiles, split_keys > 0 ? max_splits : 1);
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if ((1 << b) == page) page_shift = b;
#define XI_PB(KC, DT, NQT, GH, NWV)                                                                     \
  do {                                                                                                  \
    auto kern = dv == 16 * DT ? attn_biased_lds_kernel<KC, DT, NQT, GH, NWV, true>                      \
                              : attn_biased_lds_kernel<KC, DT, NQT, GH, NWV, false>;                    \
    const size_t lds = 2 * (size_t)(kKeysB * (32 * KC + kVPadB) + dv * (kKeysB + kVPadB)) * sizeof(bf16) + \
                       (size_t)max_pages * sizeof(int);                                                 \
    XI_CHECK(lds <= 160 * 1024, "attention_biased: block tables of %d pages do not fit in LDS", max_pages); \
    if (lds > 48 * 1024) {                                                                              \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                         (int)lds);                                                     \
      XI_CHECK(e == hipSuccess, "attention_biased: cannot get %zu bytes of LDS: %s", lds,               \
               hipGetErrorString(e));                                                                   \
    }                                                                                                   \
    kern<<<grid, 64 * NWV, lds, stream>>>((const bf16*)q, (const bf16*)k_cache, (const bf16*)vt_cache,  \
                                          block_tables, max_pages, tiles, cu_q, ctx_lens, (bf16*)out,   \
                                          scale, softcap, slopes, sinks, window, page_shift, nq, nkv, d,\
                                          dv, part_o, part_ml, split_keys, max_splits, rows_heads, nkk, rows_kv);\
  } while (0)
#define XI_PB_GH(KC, DT, NQT, NWV)             \
  do {                                         \
    if (gh == 4) XI_PB(KC, DT, NQT, 4, NWV);   \
    else if (gh == 2) XI_PB(KC, DT, NQT, 2, NWV); \
    else XI_PB(KC, DT, NQT, 1, NWV);           \
  } while (0)
#define XI_PB_DV(KC, NQT, NWV)                        \
  do {                                                \
    if (dv <= 64) XI_PB_GH(KC, 4, NQT, NWV);          \
    else if (dv <= 128) XI_PB_GH(KC, 8, NQT, NWV);    \
    else XI_PB_GH(KC, 16, NQT, NWV);                  \
  } while (0)
  const int dmax = d > dv ? d : dv;
  if (dmax <= 128) {        // two column tiles a wave
    if (small) {
      if (d <= 64) XI_PB_DV(2, 2, 4);
      else XI_PB_DV(4, 2, 4);
    } else {
      if (d <= 64) XI_PB_DV(2, 2, 8);
      else XI_PB_DV(4, 2, 8);
    }
  } else {                  // one
    if (small) {
      if (d <= 64) XI_PB_DV(2, 1, 4);
      else if (d <= 128) XI_PB_DV(4, 1, 4);
      else XI_PB_DV(8, 1, 4);
    } else {
      if (d <= 64) XI_PB_DV(2, 1, 8);
      else if (d <= 128) XI_PB_DV(4, 1, 8);
      else XI_PB_DV(8, 1, 8);
    }
  }
#undef XI_PB_DV
#undef XI_PB_GH
#undef XI_PB
  XI_LAUNCH_CHECK("attention_biased");
  if (split_keys > 0) {
    attn_biased_combine_kernel<<<dim3(nq, n_tok), 64, 0, stream>>>(part_o, part_ml, (bf16*)out, sinks, max_splits, nq, dv, rows_heads);
    XI_LAUNCH_CHECK("attention_biased_combine");
  }
  return 0;
}

}  // extern "C"
