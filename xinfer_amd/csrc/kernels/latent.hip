// Attention over a latent: what a token keeps is one vector c (rank dims, the RMS-normed first part of a down
// projection) and one rotated key part (r dims) shared by all heads; a head's keys and values are products of c
// with matrices of its own, U_k [dim, rank] and U_v [vdim, rank].  Both products move to the query's side:
//
//   score(i, j) = ((U_k^T q_plain_i) . c_j + q_turned_i . k_turned_j) * scale        o_i = U_v (sum_j p_ij c_j)
//
// so the attention itself is one kv head with keys [c | k_turned] of rank + r dims whose first `rank` dims are
// the values too, read from one pool [pages, 1, page, rank + r].  The matrix-core attention kernels read values in
// groups of eight keys, [pages, 1, page / 8, rank, 8]: where such a pool is given, c is written there once more.
//
// `latent_rows_kernel`, a workgroup a token, from the packed projection row [q (H (dim + r)) | down (rank + r) | ..]:
//   c = down[:rank] / sqrt(mean(down[:rank]^2) + eps) * w   and the turned down[rank:] into the pool at the slot;
//   every head's turned q part into q_full[t, h, rank:] (the q parts may be rows of another tensor, `q_rows`).
// Pairs (2i, 2i + 1) or (i, i + r / 2) turn by the position's row of float32 tables [positions, r / 2].
//
// `head_linear_kernel`: out[t, h, n] = sum_k x[t, h, k] * w[h][n][k] for every head, with the strides of all
// three given (U_k is read as [k][n], U_v as [n][k]); float32 sums in ascending k (a tile of 32 at a time); with a
// gate, out *= sigmoid(gate[t, h, n]).
#include "common.h"

namespace xi {

template <typename T>
__global__ __launch_bounds__(256) void latent_rows_kernel(const T* __restrict__ proj, long long proj_stride, int q_off,
                                                          int down_off, const float* __restrict__ w, float eps,
                                                          const long long* __restrict__ slots, T* __restrict__ pool,
                                                          T* __restrict__ values, int page_size, T* __restrict__ q_full, int H, int dim, int r,
                                                          int rank, const float* __restrict__ cos_t,
                                                          const float* __restrict__ sin_t, int interleaved,
                                                          const int* __restrict__ positions, const T* __restrict__ q_rows,
                                                          long long q_stride) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * proj_stride;
  const T* qrow = q_rows + (size_t)t * q_stride;       // the heads' q parts: the same rows, or rows of their own
  const int half = r / 2;
  const size_t trow = (size_t)positions[t] * half;
  // the heads' turned parts
  T* qf = q_full + (size_t)t * H * (rank + r);
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int h = i / half, p = i - h * half;
    const int ia = interleaved ? 2 * p : p, ib = interleaved ? 2 * p + 1 : p + half;
    const T* src = qrow + q_off + (size_t)h * (dim + r) + dim;
    const float a = to_float(src[ia]), b = to_float(src[ib]);
    const float cs = cos_t[trow + p], sn = sin_t[trow + p];
    T* dst = qf + (size_t)h * (rank + r) + rank;
    dst[ia] = from_float<T>(a * cs - b * sn);
    dst[ib] = from_float<T>(b * cs + a * sn);
  }
  const T* down = row + down_off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_float(down[i]);
    ss = fmaf(v, v, ss);
  }
  const float inv = rsqrtf(block_sum<4>(ss, scratch) / (float)rank + eps);
  const long long slot = slots[t];
  if (slot < 0) return;
  T* dst = pool + (size_t)slot * (rank + r);       // [pages, 1, page, rank + r]: slot = page * page_size + offset
  // values in groups of eight keys: token `off` of a page at [off / 8][i][off % 8]
  const long long pg = slot / page_size;
  const int off = (int)(slot - pg * page_size);
  T* vdst = values ? values + ((size_t)pg * (page_size / 8) + off / 8) * (size_t)rank * 8 + (off & 7) : nullptr;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const T c = from_float<T>(to_float(down[i]) * inv * w[i]);
    dst[i] = c;
    if (vdst) vdst[(size_t)i * 8] = c;
  }
  for (int p = threadIdx.x; p < half; p += blockDim.x) {
    const int ia = interleaved ? 2 * p : p, ib = interleaved ? 2 * p + 1 : p + half;
    const float a = to_float(down[rank + ia]), b = to_float(down[rank + ib]);
    const float cs = cos_t[trow + p], sn = sin_t[trow + p];
    dst[rank + ia] = from_float<T>(a * cs - b * sn);
    dst[rank + ib] = from_float<T>(b * cs + a * sn);
  }
}

constexpr int kHlRows = 32, kHlCols = 64, kHlK = 32;

// a workgroup of 256 threads: 32 tokens by 64 outputs of one head; a thread 2 tokens by 4 outputs
template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(const T* __restrict__ x, long long x_row, long long x_head,
                                                          const T* __restrict__ w, long long w_head, long long w_n,
                                                          long long w_k, T* __restrict__ out, long long o_row,
                                                          long long o_head, const T* __restrict__ gate, long long g_row,
                                                          long long g_head, int g_each, int n_tok, int N, int K) {
  __shared__ float xs[kHlK][kHlRows + 1];
  __shared__ float ws[kHlK][kHlCols + 1];
  const int h = blockIdx.z;
  const int t0 = blockIdx.x * kHlRows, n0 = blockIdx.y * kHlCols;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;       // outputs n0 + tx + 16 j, tokens t0 + ty + 16 i
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  const T* xh = x + (size_t)h * x_head;
  const T* wh = w + (size_t)h * w_head;
  for (int k0 = 0; k0 < K; k0 += kHlK) {
    for (int e = threadIdx.x; e < kHlK * kHlRows; e += 256) {
      const int tt = e / kHlK, kk = e - tt * kHlK;              // k fastest: x's k is contiguous
      const int t = t0 + tt, k = k0 + kk;
      xs[kk][tt] = (t < n_tok && k < K) ? to_float(xh[(size_t)t * x_row + k]) : 0.f;
    }
    for (int e = threadIdx.x; e < kHlK * kHlCols; e += 256) {
      int nn, kk;
      if (w_k == 1) {                                           // k contiguous
        nn = e / kHlK;
        kk = e - nn * kHlK;
      } else {                                                  // n contiguous
        kk = e / kHlCols;
        nn = e - kk * kHlCols;
      }
      const int n = n0 + nn, k = k0 + kk;
      ws[kk][nn] = (n < N && k < K) ? to_float(wh[(size_t)n * w_n + (size_t)k * w_k]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kHlK; ++kk) {
      const float a0 = xs[kk][ty], a1 = xs[kk][ty + 16];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = ws[kk][tx + 16 * j];
        acc[0][j] = fmaf(a0, b, acc[0][j]);
        acc[1][j] = fmaf(a1, b, acc[1][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int t = t0 + ty + 16 * i;
    if (t >= n_tok) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (gate) {
        const float g = to_float(gate[(size_t)t * g_row + (size_t)h * g_head + (g_each ? n : 0)]);
        v *= 1.f / (1.f + expf(-g));
      }
      out[(size_t)t * o_row + (size_t)h * o_head + n] = from_float<T>(v);
    }
  }
}

// ---- the same product on the matrix cores (bfloat16, inputs of every operand side by side) -------------------------
// A workgroup of four waves: 128 tokens by 64 outputs of one head; wave v multiplies tokens 32 v .. 32 v + 31 by all
// 64 outputs as 4 x 2 v_mfma_f32_16x16x32_bf16 tiles a 32-wide k step (A = 16 rows of w, B = 16 rows of x: a lane ends
// with 4 outputs side by side of one token).  The operands go from memory straight into the lanes that multiply them,
// a k step ahead: a wave's tokens are its own, and a head's weights are few enough to come from the caches for every
// wave.  What lies past K is zeros; rows past the last token or output read the last one again and are dropped.  An
// output's sum depends on K alone, never on the tokens beside it.
typedef __attribute__((ext_vector_type(8))) __bf16 hl_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hl_f32x4;
constexpr int kHmRows = 128, kHmCols = 64;

__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const bf16* __restrict__ x, long long x_row, long long x_head,
                                                               const bf16* __restrict__ w, long long w_head, long long w_n,
                                                               bf16* __restrict__ out, long long o_row, long long o_head,
                                                               const bf16* __restrict__ gate, long long g_row,
                                                               long long g_head, int g_each, int n_tok, int N, int K, int wide) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int h = blockIdx.z;
  const int t0 = blockIdx.x * kHmRows, n0 = blockIdx.y * kHmCols;
  const bool wave_active = t0 + 32 * wave < n_tok;           // the same for a whole wave
  if (!wave_active) return;
  const bf16* xp[2];
  const bf16* wp[4];
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    int t = t0 + 32 * wave + 16 * tj + r;
    t = t < n_tok ? t : n_tok - 1;
    xp[tj] = x + (size_t)h * x_head + (size_t)t * x_row + 8 * j;
  }
#pragma unroll
  for (int ti = 0; ti < 4; ++ti) {
    int n = n0 + 16 * ti + r;
    n = n < N ? n : N - 1;
    wp[ti] = w + (size_t)h * w_head + (size_t)n * w_n + 8 * j;
  }
  hl_f32x4 acc[4][2];
#pragma unroll
  for (int ti = 0; ti < 4; ++ti)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) acc[ti][tj] = hl_f32x4{0.f, 0.f, 0.f, 0.f};
  const hl_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  hl_bf16x8 a[4], b[2], an[4], bn[2];
  const bool first = 8 * j < K;
#pragma unroll
  for (int ti = 0; ti < 4; ++ti) a[ti] = first ? *reinterpret_cast<const hl_bf16x8*>(wp[ti]) : zero;
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) b[tj] = first ? *reinterpret_cast<const hl_bf16x8*>(xp[tj]) : zero;
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int kn = k0 + 32 + 8 * j;                           // this lane's chunk of the next step
    const bool more = kn < K;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti) an[ti] = more ? *reinterpret_cast<const hl_bf16x8*>(wp[ti] + k0 + 32) : zero;
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) bn[tj] = more ? *reinterpret_cast<const hl_bf16x8*>(xp[tj] + k0 + 32) : zero;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj) acc[ti][tj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ti], b[tj], acc[ti][tj], 0, 0, 0);
#pragma unroll
    for (int ti = 0; ti < 4; ++ti) a[ti] = an[ti];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) b[tj] = bn[tj];
  }
  // a lane's 4 values of a tile: token 16 tj + r of the wave's, outputs 16 ti + 4 j .. + 3
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    const int t = t0 + 32 * wave + 16 * tj + r;
    if (t >= n_tok) continue;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti) {
      const int nf = n0 + 16 * ti + 4 * j;
      if (wide && nf + 3 < N) {              // the lane's 4 outputs in one 8-byte store (and one load of the gate)
        float v[4] = {acc[ti][tj][0], acc[ti][tj][1], acc[ti][tj][2], acc[ti][tj][3]};
        if (gate && !g_each) {                   // one number a head
          const float sg = 1.f / (1.f + expf(-to_float(gate[(size_t)t * g_row + (size_t)h * g_head])));
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] *= sg;
        } else if (gate) {
          const uint2 gb = *reinterpret_cast<const uint2*>(gate + (size_t)t * g_row + (size_t)h * g_head + nf);
          const float g4[4] = {__uint_as_float(gb.x << 16), __uint_as_float(gb.x & 0xffff0000u), __uint_as_float(gb.y << 16),
                               __uint_as_float(gb.y & 0xffff0000u)};
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] *= 1.f / (1.f + expf(-g4[i]));
        }
        unsigned short b4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bf16 o = __float2bfloat16(v[i]);
          b4[i] = *reinterpret_cast<const unsigned short*>(&o);
        }
        *reinterpret_cast<uint2*>(out + (size_t)t * o_row + (size_t)h * o_head + nf) =
            make_uint2((unsigned)b4[0] | ((unsigned)b4[1] << 16), (unsigned)b4[2] | ((unsigned)b4[3] << 16));
        continue;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = nf + i;
        if (n >= N) continue;
        float v = acc[ti][tj][i];
        if (gate) {
          const float g = to_float(gate[(size_t)t * g_row + (size_t)h * g_head + (g_each ? n : 0)]);
          v *= 1.f / (1.f + expf(-g));
        }
        out[(size_t)t * o_row + (size_t)h * o_head + n] = from_float<bf16>(v);
      }
    }
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// proj rows of proj_stride elements: the heads' q parts [H, dim + r] from q_off, the down projection [rank + r] from
// down_off; w float32 [rank]; pool [pages, 1, page, rank + r]; q_full [T, H, rank + r] (its last r dims are written).
int xi_latent_rows(const void* proj, long long proj_stride, int q_off, int down_off, int dtype, const float* w, float eps,
                   const long long* slots, void* pool, void* values, int page_size, void* q_full, int n_tok, int H, int dim, int r, int rank,
                   const float* cos_t, const float* sin_t, int interleaved, const int* positions, const void* q_rows,
                   long long q_stride, hipStream_t stream) {
  if (q_rows == nullptr) {
    q_rows = proj;
    q_stride = proj_stride;
  }
  XI_CHECK(n_tok >= 0 && H > 0 && dim > 0 && r >= 0 && r % 2 == 0 && rank > 0 && page_size > 0,
           "latent_rows: bad sizes T=%d H=%d dim=%d r=%d rank=%d page=%d", n_tok, H, dim, r, rank, page_size);
  XI_CHECK(q_off >= 0 && down_off >= 0 && q_stride >= (long long)q_off + (long long)H * (dim + r) &&
               proj_stride >= (long long)down_off + rank + r,
           "latent_rows: the projection's rows are too short");
  XI_CHECK(r == 0 || (cos_t && sin_t), "latent_rows: a rotation needs its tables");
  XI_CHECK(w && positions && slots, "latent_rows: the norm's weight, the positions and the slots are needed");
  XI_CHECK(values == nullptr || page_size % 8 == 0, "latent_rows: values in groups of eight need pages of a multiple of 8");
  if (n_tok == 0) return 0;
  if (dtype == kF32)
    latent_rows_kernel<float><<<n_tok, 256, 0, stream>>>((const float*)proj, proj_stride, q_off, down_off, w, eps, slots,
                                                         (float*)pool, (float*)values, page_size, (float*)q_full, H, dim, r, rank, cos_t,
                                                         sin_t, interleaved, positions, (const float*)q_rows, q_stride);
  else if (dtype == kBF16)
    latent_rows_kernel<bf16><<<n_tok, 256, 0, stream>>>((const bf16*)proj, proj_stride, q_off, down_off, w, eps, slots,
                                                        (bf16*)pool, (bf16*)values, page_size, (bf16*)q_full, H, dim, r, rank, cos_t, sin_t,
                                                        interleaved, positions, (const bf16*)q_rows, q_stride);
  else
    XI_CHECK(false, "latent_rows: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("latent_rows");
  return 0;
}

// x: token t, head h, element k at x + t x_row + h x_head + k; w: head h, output n, element k at w + h w_head + n w_n +
// k w_k (one of w_n, w_k is 1); out: at out + t o_row + h o_head + n; gate null or laid out like out with its own strides,
// or (g_each 0) one number a head at gate + t g_row + h g_head.
int xi_head_linear(const void* x, long long x_row, long long x_head, const void* w, long long w_head, long long w_n,
                   long long w_k, void* out, long long o_row, long long o_head, const void* gate, long long g_row,
                   long long g_head, int g_each, int dtype, int n_tok, int H, int N, int K, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && N > 0 && K > 0, "head_linear: bad sizes T=%d H=%d N=%d K=%d", n_tok, H, N, K);
  XI_CHECK(w_n == 1 || w_k == 1, "head_linear: the weight's outputs or its inputs must lie side by side");
  XI_CHECK(H <= 65535, "head_linear: too many heads");
  if (n_tok == 0) return 0;
  dim3 grid((unsigned)((n_tok + kHlRows - 1) / kHlRows), (unsigned)((N + kHlCols - 1) / kHlCols), (unsigned)H);
  XI_CHECK(grid.y <= 65535u, "head_linear: too many outputs");
  // bfloat16 with every operand's inputs side by side in whole 16-byte chunks: the matrix cores
  const bool chunks = K % 8 == 0 && w_k == 1 && x_row % 8 == 0 && x_head % 8 == 0 && w_head % 8 == 0 && w_n % 8 == 0 &&
                      (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0;
  if (dtype == kBF16 && chunks) {
    dim3 mgrid((unsigned)((n_tok + kHmRows - 1) / kHmRows), (unsigned)((N + kHmCols - 1) / kHmCols), (unsigned)H);
    // outputs (and the gate) in 8-byte pieces where every lane's 4 outputs start at one
    const int wide = o_row % 4 == 0 && o_head % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0 &&
                     (gate == nullptr || !g_each ||
                      (g_row % 4 == 0 && g_head % 4 == 0 && (reinterpret_cast<uintptr_t>(gate) & 7) == 0));
    head_linear_mfma_kernel<<<mgrid, 256, 0, stream>>>((const bf16*)x, x_row, x_head, (const bf16*)w, w_head, w_n, (bf16*)out,
                                                       o_row, o_head, (const bf16*)gate, g_row, g_head, g_each, n_tok, N, K, wide);
    XI_LAUNCH_CHECK("head_linear");
    return 0;
  }
  if (dtype == kF32)
    head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_row, x_head, (const float*)w, w_head, w_n, w_k,
                                                        (float*)out, o_row, o_head, (const float*)gate, g_row, g_head, g_each,
                                                        n_tok, N, K);
  else if (dtype == kBF16)
    head_linear_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)x, x_row, x_head, (const bf16*)w, w_head, w_n, w_k,
                                                       (bf16*)out, o_row, o_head, (const bf16*)gate, g_row, g_head, g_each, n_tok,
                                                       N, K);
  else
    XI_CHECK(false, "head_linear: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("head_linear");
  return 0;
}

}  // extern "C"
