// Routed experts for many tokens on the gfx950 matrix cores (bfloat16): the (token, chosen expert)
// pairs are put in the order of their experts on the device, and each expert's rows go through its
// weights in tiles, so a weight is read once per tile of up to 128 rows instead of once per pair.
//
//   moe_sort      pairs [T * top] -> `order` (slot -> pair), `slot_of` (pair -> slot), and the list of
//                 tiles (expert, first slot, rows); one workgroup, nothing read on the host
//   group product out[slot, n] = sum_k A[row(slot), k] * W[expert, n, k] with v_mfma_f32_16x16x32_bf16:
//                 a workgroup of four waves owns one tile of rows and 128 output features, a wave
//                 32 of them; operands come straight from memory, 16 bytes a lane (a row's 64 bytes
//                 of a K step lie side by side), and stay in registers for MI x 2 products.
//                 Gated form: W = [gate; up] rows, result act(gate) * up in bfloat16 (the experts'
//                 hidden rows, kept in slot order); activated form: W the up rows alone, result
//                 act(up) in bfloat16 (experts without a gate); plain form: float32.
//   moe_combine   out[t] = sum over the token's chosen experts, in the order they were chosen, of
//                 weight * row: a fixed order, float32.
// A row's result depends on its own operands alone (the matrix cores keep rows apart), so it does not
// matter which other rows share its tile.
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 mbf16x8;
typedef __attribute__((ext_vector_type(4))) float mf32x4;

constexpr int kSortThreads = 1024;
constexpr int kSortExperts = 1024;

__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(const int* __restrict__ idx, int P, int E, int BM,
                                                                int* __restrict__ order, int* __restrict__ slot_of,
                                                                int* __restrict__ tile_expert, int* __restrict__ tile_row0,
                                                                int* __restrict__ tile_rows, int* __restrict__ n_tiles) {
  __shared__ int count[kSortExperts], cursor[kSortExperts];
  for (int e = threadIdx.x; e < E; e += kSortThreads) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += kSortThreads) {
    int e = idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      cursor[e] = at;
      for (int r = 0; r < count[e]; r += BM) {
        tile_expert[tiles] = e;
        tile_row0[tiles] = at + r;
        tile_rows[tiles] = count[e] - r < BM ? count[e] - r : BM;
        ++tiles;
      }
      at += count[e];
    }
    *n_tiles = tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += kSortThreads) {
    int e = idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    const int slot = atomicAdd(&cursor[e], 1);
    order[slot] = p;
    slot_of[p] = slot;
  }
}

template <int ACT>
__device__ __forceinline__ float moe_act_m(float z) {
  if constexpr (ACT == 2) return z > 0.f ? z * z : 0.f;       // the square of relu
  if constexpr (ACT == 0) return z / (1.f + __expf(-z));
  else return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

static __device__ __forceinline__ mbf16x8 mld8(const bf16* p) { return *reinterpret_cast<const mbf16x8*>(p); }
static __device__ __forceinline__ mbf16x8 mzero8() {
  mbf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// MI: row tiles of 16 a workgroup (its tile has up to 16 * MI rows).  FORM: 0 plain, 1 gated, 2 activated (see
// the head of the file); the last two read their rows from x through `order`.
template <int MI, int FORM, int ACT>
__global__ __launch_bounds__(256) void moe_group_kernel(const bf16* __restrict__ A, const int* __restrict__ order, int top,
                                                        const bf16* __restrict__ W, const int* __restrict__ tile_expert,
                                                        const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
                                                        const int* __restrict__ n_tiles, void* __restrict__ out, int N,
                                                        int K, const float* __restrict__ in_wt) {
  constexpr bool GATED = FORM == 1, GATHER = FORM != 0;
  const int tile = blockIdx.x;
  if (tile >= *n_tiles) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile], rows = tile_rows[tile];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int nw0 = blockIdx.y * 128 + wave * 32;
  if (nw0 >= N) return;
  const bf16* ap[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    int slot = row0 + 16 * i + r;
    slot = slot < row0 + rows ? slot : row0 + rows - 1;
    const size_t arow = GATHER ? (size_t)(order[slot] / top) : (size_t)slot;
    ap[i] = A + arow * K;
  }
  constexpr int NB = GATED ? 4 : 2;
  const bf16* bp[NB];
  const bf16* We = W + (size_t)e * (GATED ? 2 : 1) * N * K;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    int col = nw0 + 16 * c + r;
    col = col < N ? col : N - 1;
    bp[c] = We + (size_t)col * K;
    if (GATED) bp[2 + c] = We + (size_t)(N + col) * K;
  }
  mf32x4 acc[MI][NB];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int c = 0; c < NB; ++c) acc[i][c] = mf32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int kk = k0 + 8 * j;
    const bool in = kk < K;
    mbf16x8 a[MI], b[NB];
#pragma unroll
    for (int i = 0; i < MI; ++i) a[i] = in ? mld8(ap[i] + kk) : mzero8();
#pragma unroll
    for (int c = 0; c < NB; ++c) b[c] = in ? mld8(bp[c] + kk) : mzero8();
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int c = 0; c < NB; ++c) acc[i][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[c], acc[i][c], 0, 0, 0);
  }
  // lane (r, j), element v of acc[i][c]: row 16 i + 4 j + v of the tile, feature nw0 + 16 c + r
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = 16 * i + 4 * j + v;
      if (row >= rows) continue;
      // a weight on the expert's INPUT: the products are linear, so it multiplies their sums before the activation
      const float wi = (GATHER && in_wt) ? in_wt[order[row0 + row]] : 1.f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int col = nw0 + 16 * c + r;
        if (col >= N) continue;
        const size_t at = (size_t)(row0 + row) * N + col;
        if (GATED)
          reinterpret_cast<bf16*>(out)[at] = __float2bfloat16(moe_act_m<ACT>(wi * acc[i][c][v]) * (wi * acc[i][GATED ? 2 + c : c][v]));
        else if (FORM == 2)
          reinterpret_cast<bf16*>(out)[at] = __float2bfloat16(moe_act_m<ACT>(wi * acc[i][c][v]));
        else
          reinterpret_cast<float*>(out)[at] = acc[i][c][v];
      }
    }
}

// The same product for tiles of up to 128 rows (experts with many rows): the rows' operand goes through LDS, read
// from memory once a workgroup instead of once a wave (two buffers, one barrier a K step; a row of 32 k is padded
// by 16 bytes against bank conflicts), the weights' operand stays with the wave that owns its features, and every
// operand of a K step feeds 8 x NB products.  The next step's loads are in flight while this one is multiplied.
template <int FORM, int ACT>
__global__ __launch_bounds__(256) void moe_group_lds_kernel(const bf16* __restrict__ A, const int* __restrict__ order, int top,
                                                            const bf16* __restrict__ W, const int* __restrict__ tile_expert,
                                                            const int* __restrict__ tile_row0,
                                                            const int* __restrict__ tile_rows, const int* __restrict__ n_tiles,
                                                            void* __restrict__ out, int N, int K,
                                                            const float* __restrict__ in_wt) {
  constexpr int MI = 8, BM = 128, LDA = 32 + 8;
  __shared__ __align__(16) bf16 As[2][BM * LDA];
  constexpr bool GATED = FORM == 1, GATHER = FORM != 0;
  const int tile = blockIdx.x;
  if (tile >= *n_tiles) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile], rows = tile_rows[tile];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int nw0 = blockIdx.y * 128 + wave * 32;
  const bool owns = nw0 < N;                 // (a wave without features still copies rows and meets the barriers)
  const bf16* agp[2];
  int adst[2], ach[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 256 * i, row = idx >> 2;
    ach[i] = 8 * (idx & 3);
    int slot = row0 + row;
    slot = slot < row0 + rows ? slot : row0 + rows - 1;
    const size_t arow = GATHER ? (size_t)(order[slot] / top) : (size_t)slot;
    agp[i] = A + arow * K + ach[i];
    adst[i] = row * LDA + ach[i];
  }
  constexpr int NB = GATED ? 4 : 2;
  const bf16* bp[NB];
  const bf16* We = W + (size_t)e * (GATED ? 2 : 1) * N * K;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    int col = nw0 + 16 * c + r;
    col = col < N ? col : N - 1;
    bp[c] = We + (size_t)col * K + 8 * j;
    if (GATED) bp[2 + c] = We + (size_t)(N + col) * K + 8 * j;
  }
  mf32x4 acc[MI][NB];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int c = 0; c < NB; ++c) acc[i][c] = mf32x4{0.f, 0.f, 0.f, 0.f};
  mbf16x8 an[2], b[NB], bn[NB];
#pragma unroll
  for (int i = 0; i < 2; ++i) an[i] = ach[i] < K ? mld8(agp[i]) : mzero8();
#pragma unroll
  for (int c = 0; c < NB; ++c) b[c] = 8 * j < K ? mld8(bp[c]) : mzero8();
#pragma unroll
  for (int i = 0; i < 2; ++i) *reinterpret_cast<mbf16x8*>(&As[0][adst[i]]) = an[i];
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool next = k0 + 32 < K;
    if (next) {
#pragma unroll
      for (int i = 0; i < 2; ++i) an[i] = k0 + 32 + ach[i] < K ? mld8(agp[i] + k0 + 32) : mzero8();
#pragma unroll
      for (int c = 0; c < NB; ++c) bn[c] = k0 + 32 + 8 * j < K ? mld8(bp[c] + k0 + 32) : mzero8();
    }
    if (owns) {
      mbf16x8 a[MI];
#pragma unroll
      for (int i = 0; i < MI; ++i) a[i] = *reinterpret_cast<const mbf16x8*>(&As[buf][(16 * i + r) * LDA + 8 * j]);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int c = 0; c < NB; ++c) acc[i][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[c], acc[i][c], 0, 0, 0);
    }
    if (next) {
#pragma unroll
      for (int i = 0; i < 2; ++i) *reinterpret_cast<mbf16x8*>(&As[buf ^ 1][adst[i]]) = an[i];
#pragma unroll
      for (int c = 0; c < NB; ++c) b[c] = bn[c];
    }
    __syncthreads();
    buf ^= 1;
  }
  if (!owns) return;
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = 16 * i + 4 * j + v;
      if (row >= rows) continue;
      // a weight on the expert's INPUT: the products are linear, so it multiplies their sums before the activation
      const float wi = (GATHER && in_wt) ? in_wt[order[row0 + row]] : 1.f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int col = nw0 + 16 * c + r;
        if (col >= N) continue;
        const size_t at = (size_t)(row0 + row) * N + col;
        if (GATED)
          reinterpret_cast<bf16*>(out)[at] = __float2bfloat16(moe_act_m<ACT>(wi * acc[i][c][v]) * (wi * acc[i][GATED ? 2 + c : c][v]));
        else if (FORM == 2)
          reinterpret_cast<bf16*>(out)[at] = __float2bfloat16(moe_act_m<ACT>(wi * acc[i][c][v]));
        else
          reinterpret_cast<float*>(out)[at] = acc[i][c][v];
      }
    }
}

__global__ void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ slot_of, const float* __restrict__ wt,
                                   float* __restrict__ out, int H, int top) {
  const int t = blockIdx.x;
  for (int n = threadIdx.x; n < H; n += blockDim.x) {
    float total = 0.f;
    for (int r = 0; r < top; ++r) total += wt[(size_t)t * top + r] * y[(size_t)slot_of[(size_t)t * top + r] * H + n];
    out[(size_t)t * H + n] = total;
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// Most tiles of up to `bm` rows that P pairs on E experts can make.
int xi_moe_tiles_most(int P, int E, int bm) { return (P + bm - 1) / bm + E; }

// idx int32 [P] (expert of every pair) -> order, slot_of int32 [P]; tile_* int32 [xi_moe_tiles_most]; n_tiles int32 [1].
int xi_moe_sort(const int* idx, int P, int E, int bm, int* order, int* slot_of, int* tile_expert, int* tile_row0,
                int* tile_rows, int* n_tiles, hipStream_t stream) {
  XI_CHECK(P > 0 && E > 0 && E <= kSortExperts && (bm == 32 || bm == 64 || bm == 128), "moe_sort: bad sizes pairs=%d experts=%d rows=%d", P, E, bm);
  moe_sort_kernel<<<1, kSortThreads, 0, stream>>>(idx, P, E, bm, order, slot_of, tile_expert, tile_row0, tile_rows, n_tiles);
  XI_LAUNCH_CHECK("moe_sort");
  return 0;
}

// form 1 (gated): A = x [T, K] (row of a slot: order[slot] / top), W [E, 2N, K], out bfloat16 [P, N] = act(gate) * up;
// form 2 (activated): the same rows, W [E, N, K], out bfloat16 [P, N] = act(up);
// form 0 (plain): A [P, K] in slot order, W [E, N, K], out float32 [P, N].  K a multiple of 8.
// act: 0 silu, 1 gelu (tanh form), 2 the square of relu.  in_wt (forms 1 and 2; null: none): float32 [P], a weight a pair
// that multiplies the expert's input.
int xi_moe_group(const void* A, const int* order, int top, const void* W, const int* tile_expert, const int* tile_row0,
                 const int* tile_rows, const int* n_tiles, int tiles_most, void* out, int N, int K, int bm, int form, int act,
                 const float* in_wt, hipStream_t stream) {
  XI_CHECK(N > 0 && K > 0 && K % 8 == 0 && top > 0 && tiles_most > 0 && (bm == 32 || bm == 64 || bm == 128),
           "moe_group: bad sizes N=%d K=%d (a multiple of 8) top=%d tiles=%d rows=%d", N, K, top, tiles_most, bm);
  XI_CHECK(act >= 0 && act <= 2 && form >= 0 && form <= 2, "moe_group: unknown activation %d or form %d", act, form);
  dim3 grid((unsigned)tiles_most, (unsigned)((N + 127) / 128));
  XI_CHECK(grid.y <= 65535u, "moe_group: N=%d is too large", N);
#define XI_MG(MI, G, ACT_)                                                                                            \
  moe_group_kernel<MI, G, ACT_><<<grid, 256, 0, stream>>>((const bf16*)A, order, top, (const bf16*)W, tile_expert,    \
                                                          tile_row0, tile_rows, n_tiles, out, N, K, in_wt)
#define XI_ML(G, ACT_)                                                                                                \
  moe_group_lds_kernel<G, ACT_><<<grid, 256, 0, stream>>>((const bf16*)A, order, top, (const bf16*)W, tile_expert,    \
                                                          tile_row0, tile_rows, n_tiles, out, N, K, in_wt)
#define XI_FORMS(LAUNCH, ...)                        \
  do {                                               \
    if (form == 0) LAUNCH(__VA_ARGS__ 0, 0);         \
    else if (form == 1 && act == 0) LAUNCH(__VA_ARGS__ 1, 0); \
    else if (form == 1 && act == 1) LAUNCH(__VA_ARGS__ 1, 1); \
    else if (form == 1) LAUNCH(__VA_ARGS__ 1, 2);    \
    else if (act == 0) LAUNCH(__VA_ARGS__ 2, 0);     \
    else if (act == 1) LAUNCH(__VA_ARGS__ 2, 1);     \
    else LAUNCH(__VA_ARGS__ 2, 2);                   \
  } while (0)
#define XI_MG2(G, ACT_) XI_MG(2, G, ACT_)
#define XI_MG4(G, ACT_) XI_MG(4, G, ACT_)
  if (bm == 128) XI_FORMS(XI_ML);
  else if (bm == 32) XI_FORMS(XI_MG2);
  else XI_FORMS(XI_MG4);
#undef XI_MG2
#undef XI_MG4
#undef XI_FORMS
#undef XI_ML
#undef XI_MG
  XI_LAUNCH_CHECK("moe_group");
  return 0;
}

// y float32 [P, H] in slot order -> out float32 [T, H]
int xi_moe_combine(const float* y, const int* slot_of, const float* wt, float* out, int n_tok, int H, int top,
                   hipStream_t stream) {
  XI_CHECK(n_tok > 0 && H > 0 && top > 0, "moe_combine: bad sizes T=%d H=%d top=%d", n_tok, H, top);
  moe_combine_kernel<<<n_tok, 256, 0, stream>>>(y, slot_of, wt, out, H, top);
  XI_LAUNCH_CHECK("moe_combine");
  return 0;
}

}  // extern "C"
