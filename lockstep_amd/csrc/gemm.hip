// C[M,N] = X[M,K] * W[N,K]^T with a fixed summation order per output element.
//
// The order, for every (m, n), whatever M is and whichever kernel runs:
//   K is cut into slices of `kslice` elements (a function of K alone);
//   inside a slice the products are accumulated by a chain of MFMA atoms over
//   ascending 64-byte chunks of K, starting from zero;
//   the slice sums are added in ascending order to a total that starts at +0.
// The skinny kernel (M <= 64, decode) gives each slice to a wave, so the
// weights stream from HBM with many waves in flight; the streaming kernel
// does the same for products with many columns, one workgroup walking many
// column blocks; the slice kernels leave the slice sums to their consumer; the
// tiled kernel (prefill) walks the slices one after the other with both
// operands staged in LDS, or (slice sums of 17 rows and more) a group of them
// a workgroup.  All produce the same bits for a row, so a token's
// projections do not depend on how many tokens share its step.
//
// The MFMA runs "swapped": W rows are the first operand, X rows the second,
// so a lane ends with four consecutive n of one row m and stores them as one
// vector.

#include <algorithm>
#include <type_traits>

#include "common.h"
#include "core_api.h"

namespace ls {

#ifndef LS_GEMM_BIG
#define LS_GEMM_BIG 0         // from this many 128 x 128 tiles on, use them; 0: one for every CU (fewer leave CUs idle and 64 x 64 tiles win)
#endif
#ifndef LS_GEMM_BIG_ROWS
#define LS_GEMM_BIG_ROWS 64   // ... and only with more rows than this: up to 64 rows half of a 128-row tile would be idle
#endif
#ifndef LS_GEMM_PD_BIG
#define LS_GEMM_PD_BIG 1      // register prefetch depth (stages) of the 128 x 128 kernel (2: registers run out, a third slower)
#endif
#ifndef LS_GEMM_SLICES_WIDE
#define LS_GEMM_SLICES_WIDE 1       // 0: never the wide slice kernel
#endif
#ifndef LS_GEMM_SLICES_WIDE_WGS
#define LS_GEMM_SLICES_WIDE_WGS 192  // its workgroups (64 columns, up to four slices) must be at least this many
#endif
#ifndef LS_GEMM_SLICES_WIDE_UNR
#define LS_GEMM_SLICES_WIDE_UNR 2   // chunks it loads at a time
#endif
#ifndef LS_GEMM_STREAM
#define LS_GEMM_STREAM 1      // 0: never the streaming kernel
#endif
#ifndef LS_GEMM_GROUP_M
#define LS_GEMM_GROUP_M 4     // row tiles per band of the tile numbering (0: column-major numbering)
#endif
#ifndef LS_GEMM_WIDE
#define LS_GEMM_WIDE 1        // 0: never the 128 x 256 tiles of eight waves
#endif
#ifndef LS_GEMM_WIDE_FILL
#define LS_GEMM_WIDE_FILL 85  // ... which need whole rounds of the CUs (one workgroup a CU): at least this share, in percent,
#endif                        // of the last round's CUs busy, or eight rounds and more
#ifndef LS_GEMM_PD_WIDE
#define LS_GEMM_PD_WIDE 2     // their register prefetch depth (2 is 1 to 4 % ahead of 1)
#endif
#ifndef LS_GEMM_READ_AHEAD
#define LS_GEMM_READ_AHEAD 1  // the tiled kernel reads a stage's second chunk of fragments from LDS before it multiplies the first
#endif
#ifndef LS_GEMM_SLICES_TILED
#define LS_GEMM_SLICES_TILED 1      // 0: never the tiled kernel for slice sums
#endif
#ifndef LS_GEMM_NARROW
#define LS_GEMM_NARROW 1      // 0: never the 64 x 32 tiles
#endif
#ifndef LS_GEMM_ROWS64_WIDE
#define LS_GEMM_ROWS64_WIDE 1 // 0: never 64 x 128 tiles for products of up to 64 rows
#endif
#ifndef LS_GEMM_PD_SMALL
#define LS_GEMM_PD_SMALL 4    // ... and of the 64 x 64 kernel (measured 1 to 4: 4 is 2 to 10 % ahead of 2)
#endif

enum Epilogue : int {
  kStore = 0,     // C[m][n] = total, in the compute dtype
  kStoreF32 = 1,  // C[m][n] = total, float
  kAddF32 = 2,    // C[m][n] += total, float (residual stream)
  kSwiGLU = 3,    // W holds gate and up rows interleaved in tiles of 16 (gate rows 16t.., then up rows 16t..);
                  // C[m][16t + i] = (g * 1/(1 + exp(-g))) * u in float, stored in the compute dtype
  kSliceSums = 4, // the tiled kernel only: C is float [slices][M][N] and gets the sums of the K slices, not their
                  // total; the workgroups with blockIdx.y = y take the slices [y * out_cols, (y + 1) * out_cols)
};

__host__ __device__ inline int kslice_for(int K) { return 256 * ((K + 4095) / 4096); }

// `old`: for kAddF32 with vector stores, the four values the element's owner
// has already read from C (nullptr: read them here).
template <typename T, int EPI>
__device__ __forceinline__ void epilogue4(void* __restrict__ C, long ldc, int m, int n, int M, int N,
                                          const float total[4], bool vec_ok, const f32x4* old_vals = nullptr) {
  if (m >= M || n >= N) return;
  if (EPI == kStore) {
    T* row = reinterpret_cast<T*>(C) + (long)m * ldc;
    if (vec_ok && n + 3 < N) {
      if (sizeof(T) == 2) {
        bf16x4 v;
        v[0] = (bf16_t)total[0]; v[1] = (bf16_t)total[1]; v[2] = (bf16_t)total[2]; v[3] = (bf16_t)total[3];
        *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(C) + (long)m * ldc + n) = v;
      } else {
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(C) + (long)m * ldc + n) =
            f32x4{total[0], total[1], total[2], total[3]};
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) row[n + r] = from_f32<T>(total[r]);
    }
  } else {
    float* row = reinterpret_cast<float*>(C) + (long)m * ldc;
    if (vec_ok && n + 3 < N) {
      f32x4* p = reinterpret_cast<f32x4*>(row + n);
      f32x4 v = f32x4{total[0], total[1], total[2], total[3]};
      if (EPI == kAddF32) {
        const f32x4 old = old_vals ? *old_vals : *p;
        v = f32x4{old[0] + v[0], old[1] + v[1], old[2] + v[2], old[3] + v[3]};
      }
      *p = v;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) row[n + r] = (EPI == kAddF32) ? row[n + r] + total[r] : total[r];
    }
  }
}

// SwiGLU epilogue on the float totals of a gate tile and the matching up tile.
template <typename T>
__device__ __forceinline__ void epilogue_swiglu4(void* __restrict__ C, long ldc, int m, int col, int M, int width,
                                                 const float gate[4], const float up[4], bool vec_ok) {
  if (m >= M || col >= width) return;
  float act[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float sig = 1.0f / (1.0f + expf(-gate[r]));
    act[r] = (gate[r] * sig) * up[r];
  }
  epilogue4<T, kStore>(C, ldc, m, col, M, width, act, vec_ok);
}

// RMSNorm of rows of the float residual stream, as a prologue of the skinny
// kernel (at most 16 rows): the sum of squares of a row is formed exactly as
// rmsnorm_kernel forms it (row_sumsq_part over the first 256 threads, a
// butterfly over the wave, the four wave sums in wave order), so the
// normalised operand has the same bits as the stand-alone kernel's.
template <int NW>
__device__ __forceinline__ void row_scales(const float* __restrict__ H, long ldh, int M, int K, float eps,
                                           float* __restrict__ wave_part /*[16][4]*/, float* __restrict__ scale /*[16]*/) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (wave < 4) {
    const bool vec_ok = (ldh & 3) == 0 && (reinterpret_cast<uintptr_t>(H) & 15) == 0;
    // four rows at a time, so that their loads are in flight together
    for (int m0 = 0; m0 < M; m0 += 4) {
      float part[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        part[j] = row_sumsq_part(H + (long)min(m0 + j, M - 1) * ldh, K, threadIdx.x, vec_ok);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float total = wave_sum(part[j]);
        if (lane == 0 && m0 + j < M) wave_part[(m0 + j) * 4 + wave] = total;
      }
    }
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    const float* p = wave_part + threadIdx.x * 4;
    const float total = ((p[0] + p[1]) + p[2]) + p[3];
    scale[threadIdx.x] = 1.0f / sqrtf(total / (float)K + eps);
  }
  __syncthreads();
}

// ---------------------------------------------------------------------------
// Skinny kernel: one workgroup per 16 output columns, NW waves, wave w takes
// slices w, w + NW, ...; slice sums meet in LDS and are folded in ascending
// order by the thread that owns the output element.
// ---------------------------------------------------------------------------
template <typename T, int MT, int NW, int EPI, bool NORM>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const void* __restrict__ Xv, const T* __restrict__ W,
                                                               void* __restrict__ C, int M, int N, int K, long ldx,
                                                               long ldc, int kslice, int aligned, int vec_ok,
                                                               const float* __restrict__ norm_w, float eps,
                                                               int out_cols) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int NT = (EPI == kSwiGLU) ? 2 : 1;  // weight tiles per workgroup
  extern __shared__ float part[];                // [nslices][NT][MT][256] (+ 80 floats with NORM)

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16 * NT;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int nslices = (K + kslice - 1) / kslice;

  const T* X = reinterpret_cast<const T*>(Xv);
  const float* H = reinterpret_cast<const float*>(Xv);
  // UNR chunks at a time: all their loads are issued before the first MFMA
  // needs one, so a wave keeps several kilobytes in flight.
  // as many chunks as the registers of a wave allow (512 / (NW / 4) a lane), so that a slice of 256 elements is one round
  constexpr int UNR = ((NT + MT) * 8 * 4 + NT * MT * 4 + 32 <= 2048 / NW && !NORM) ? 8 : 4;
  auto load_w = [&](int k0, int k_end, vec_t (&w)[NT][UNR]) LS_INLINED {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * A::KCHUNK + g * A::VEC;
      const bool in = k0 + u * A::KCHUNK < k_end;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int n = n0 + t * 16 + row16;
        w[t][u] = load_vec<T>(W, n, k, K, K, n < N && in, aligned);
      }
    }
  };
  float my_scale = 0.f;
  vec_t w_first[NT][UNR];  // with NORM: the wave's first weights are in flight while the rows are reduced
  if (NORM) {
    if (wave < nslices) load_w(wave * kslice, min(K, (wave + 1) * kslice), w_first);
    float* wave_part = part + nslices * NT * MT * 256;
    float* scale = wave_part + 64;
    row_scales<NW>(H, ldx, M, K, eps, wave_part, scale);
    my_scale = row16 < M ? scale[row16] : 0.f;
  }
  const bool norm_vec = NORM && aligned && ldx % 4 == 0 && reinterpret_cast<uintptr_t>(norm_w) % 16 == 0;

  // kAddF32: the owner of an output element reads its old value now, not after the products
  f32x4 old_vals = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool preload = EPI == kAddF32 && vec_ok && (int)threadIdx.x < MT * 64 &&
                       (int)(threadIdx.x >> 6) * 16 + row16 < M && n0 + g * 4 + 3 < N;
  if (preload)
    old_vals = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(C) +
                                               (long)((threadIdx.x >> 6) * 16 + row16) * ldc + n0 + g * 4);

  for (int s = wave; s < nslices; s += NW) {
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int j = 0; j < MT; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int k_begin = s * kslice;
    const int k_end = min(K, k_begin + kslice);
    for (int k0 = k_begin; k0 < k_end; k0 += UNR * A::KCHUNK) {
      vec_t w[NT][UNR], x[MT][UNR];
      if (NORM && s == wave && k0 == k_begin) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int u = 0; u < UNR; ++u) w[t][u] = w_first[t][u];
      } else {
        load_w(k0, k_end, w);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int k = k0 + u * A::KCHUNK + g * A::VEC;
        const bool in = k0 + u * A::KCHUNK < k_end;
        if (NORM) {
          // normalise on the fly: (x * scale) * weight, rounded to the compute dtype
          vec_t v = A::zero();
          const bool valid = row16 < M && in && k < K;
          if (norm_vec) {  // uniform: rows and k are 16-byte aligned and K is a multiple of VEC
            const float* src = H + (valid ? (long)row16 * ldx + k : 0);
            const float* wsrc = norm_w + (valid ? k : 0);
#pragma unroll
            for (int q4 = 0; q4 < A::VEC / 4; ++q4) {
              const f32x4 xs = *reinterpret_cast<const f32x4*>(src + 4 * q4);
              const f32x4 ws = *reinterpret_cast<const f32x4*>(wsrc + 4 * q4);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[4 * q4 + e] = from_f32<T>((xs[e] * my_scale) * ws[e]);
            }
            if (!valid) v = A::zero();
          } else if (valid) {
            const float* src = H + (long)row16 * ldx + k;
#pragma unroll
            for (int e = 0; e < A::VEC; ++e)
              if (k + e < K) v[e] = from_f32<T>((src[e] * my_scale) * norm_w[k + e]);
          }
          x[0][u] = v;
        } else {
#pragma unroll
          for (int j = 0; j < MT; ++j)
            x[j][u] = load_vec<T>(X, j * 16 + row16, k, K, ldx, j * 16 + row16 < M && in, aligned);
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        if (k0 + u * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int j = 0; j < MT; ++j) A::mma(acc[t][j], w[t][u], x[j][u]);
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int j = 0; j < MT; ++j)
        *reinterpret_cast<f32x4*>(&part[(((s * NT + t) * MT + j) * 64 + lane) * 4]) = acc[t][j];
  }
  __syncthreads();

  for (int idx = threadIdx.x; idx < MT * 64; idx += NW * 64) {
    const int j = idx >> 6;
    const int l = idx & 63;
    float total[NT][4];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int r = 0; r < 4; ++r) total[t][r] = 0.f;
      for (int s = 0; s < nslices; ++s) {
        f32x4 p = *reinterpret_cast<const f32x4*>(&part[(((s * NT + t) * MT + j) * 64 + l) * 4]);
#pragma unroll
        for (int r = 0; r < 4; ++r) total[t][r] = total[t][r] + p[r];
      }
    }
    const int m = j * 16 + (l & 15);
    if (EPI == kSwiGLU)
      epilogue_swiglu4<T>(C, ldc, m, blockIdx.x * 16 + (l >> 4) * 4, M, out_cols, total[0], total[NT - 1], vec_ok);
    else
      epilogue4<T, EPI>(C, ldc, m, n0 + (l >> 4) * 4, M, N, total[0], vec_ok,
                        (preload && idx == (int)threadIdx.x) ? &old_vals : nullptr);
  }
}

// ---------------------------------------------------------------------------
// Streaming kernel (at most 32 rows, many output columns): the skinny kernel's
// arithmetic with another walk.  A workgroup has one wave per K slice and
// takes the column blocks b = blockIdx.x, blockIdx.x + gridDim.x, ...  A wave
// keeps its slice of X in registers for the whole walk, so the rows of X are
// read once per workgroup instead of once per 16 columns (with 8 rows that is
// half as much again as the weights themselves), and the weights of its next
// unit (UC chunks of a tile) are always in flight while it multiplies the
// current one, also across column blocks and across the two barriers of the
// fold.  Slice sums meet in LDS and are folded in ascending order, as in the
// skinny kernel.
// ---------------------------------------------------------------------------
template <typename T, int MT, int EPI, int XC>
__global__ __launch_bounds__(1024) void gemm_stream_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                           void* __restrict__ C, int M, int N, int K, long ldx,
                                                           long ldc, int kslice, int aligned, int vec_ok,
                                                           int out_cols, int blocks, int row_groups) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int NT = (EPI == kSwiGLU) ? 2 : 1;  // weight tiles per column block
  constexpr int UC = 4;                          // chunks per unit
  constexpr int UQ = XC / UC;                    // units per tile
  constexpr int UNITS = NT * UQ;                 // units per column block
  constexpr int RING = (MT * XC <= 8) ? 4 : 2;   // unit buffers in registers: one in use, the others in flight
  constexpr int AHEAD = RING - 1;
  static_assert(XC % UC == 0, "a tile is a whole number of units");
  extern __shared__ float part[];  // [2][waves][NT][MT][256]

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;  // = number of K slices
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int k_begin = wave * kslice;
  const int k_end = min(K, k_begin + kslice);
  // With more than 16 * MT rows the rows are cut into groups of 16 * MT, each with workgroups of its own
  // that walk the same column blocks.  Workgroup ids go round the XCDs, so the ids 8i .. 8i + 7 of one group
  // and the next eight ids of the other group sit pairwise on the same XCD and walk in step: what one of
  // them has fetched, the other finds in that XCD's L2.
  const int id = blockIdx.x;
  const int row_group = row_groups > 1 ? (id >> 3) % row_groups : 0;
  const int walker = row_groups > 1 ? (id / (8 * row_groups)) * 8 + (id & 7) : id;
  const int walkers = gridDim.x / row_groups;
  const int m_base = row_group * MT * 16;

  auto fetch = [&](int b, int t, int q, vec_t (&dst)[UC]) LS_INLINED {
    const int n = (b * NT + t) * 16 + row16;
#pragma unroll
    for (int c = 0; c < UC; ++c) {
      const int kc = k_begin + (q * UC + c) * A::KCHUNK;
      dst[c] = load_vec<T>(W, n, kc + g * A::VEC, K, K, n < N && kc < k_end, aligned);
    }
  };

  // Units are numbered through the walk: unit u of the workgroup is unit u % UNITS of its block u / UNITS
  // and lives in buffer u % RING.
  vec_t wbuf[RING][UC];
  int b = walker;
#pragma unroll
  for (int u = 0; u < AHEAD; ++u) {
    const int bu = b + (u / UNITS) * walkers;
    if (bu < blocks) fetch(bu, (u % UNITS) / UQ, (u % UNITS) % UQ, wbuf[u % RING]);
  }

  vec_t xs[MT][XC];
#pragma unroll
  for (int j = 0; j < MT; ++j)
#pragma unroll
    for (int c = 0; c < XC; ++c) {
      const int kc = k_begin + c * A::KCHUNK;
      xs[j][c] = load_vec<T>(X, m_base + j * 16 + row16, kc + g * A::VEC, K, ldx,
                             m_base + j * 16 + row16 < M && kc < k_end, aligned);
    }

  // One column block; `par` is the buffer that holds the block's first unit (static, so that the
  // register buffers are addressed statically).
  static_assert(UNITS % RING == 0 || (2 * UNITS) % RING == 0, "the buffer of a block's first unit has period two");
  auto block_step = [&](auto par, int it) LS_INLINED {
    constexpr int P = decltype(par)::value;
    float* mine = part + (it & 1) * (nw * NT * MT * 256);
    f32x4 acc[MT];  // of the tile in work; a finished tile's sums go to LDS at once
#pragma unroll
    for (int idx = 0; idx < UNITS; ++idx) {
      const int t = idx / UQ;
      const int q = idx % UQ;
      if (q == 0) {
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      const int far_block = b + ((idx + AHEAD) / UNITS) * walkers;  // the block of the unit AHEAD units on
      if (far_block < blocks)
        fetch(far_block, ((idx + AHEAD) % UNITS) / UQ, ((idx + AHEAD) % UNITS) % UQ, wbuf[(P + idx + AHEAD) % RING]);
#pragma unroll
      for (int c = 0; c < UC; ++c) {
        if (k_begin + (q * UC + c) * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
        for (int j = 0; j < MT; ++j) A::mma(acc[j], wbuf[(P + idx) % RING][c], xs[j][q * UC + c]);
      }
      if (q == UQ - 1) {
#pragma unroll
        for (int j = 0; j < MT; ++j)
          *reinterpret_cast<f32x4*>(&mine[(((wave * NT + t) * MT + j) * 64 + lane) * 4]) = acc[j];
      }
    }
    // One barrier a block: the next block's sums go to the other half of `part`, and the half
    // written now is written again only after the next barrier, which the folding wave reaches
    // after its fold.
    __syncthreads();
    // row tile j of this block is folded by wave (it * MT + j) % nw, so the duty goes round
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      if ((it * MT + j) % nw != wave) continue;  // uniform for the wave
      float total[NT][4];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) total[t][r] = 0.f;
        for (int s = 0; s < nw; ++s) {
          const f32x4 p = *reinterpret_cast<const f32x4*>(&mine[(((s * NT + t) * MT + j) * 64 + lane) * 4]);
#pragma unroll
          for (int r = 0; r < 4; ++r) total[t][r] = total[t][r] + p[r];
        }
      }
      const int m = m_base + j * 16 + row16;
      if (EPI == kSwiGLU)
        epilogue_swiglu4<T>(C, ldc, m, b * 16 + g * 4, M, out_cols, total[0], total[NT - 1], vec_ok);
      else
        epilogue4<T, EPI>(C, ldc, m, b * 16 + g * 4, M, N, total[0], vec_ok);
    }
  };

  // the first buffer of a block advances by UNITS % RING from block to block
  for (int it = 0; b < blocks;) {
    block_step(std::integral_constant<int, 0>{}, it);
    b += walkers;
    ++it;
    if (UNITS % RING != 0) {  // UNITS = 2, RING = 4: every other block starts in buffer 2
      if (b >= blocks) break;
      block_step(std::integral_constant<int, UNITS % RING>{}, it);
      b += walkers;
      ++it;
    }
  }
}

// Dynamic LDS beyond 64 KB has to be granted per kernel (once).
template <typename T, int MT, int EPI, int XC>
static bool stream_lds_ready(size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  if (bytes > 128 * 1024) return false;
  static int state = 0;  // 0 unknown, 1 granted, -1 refused
  if (state == 0) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_stream_kernel<T, MT, EPI, XC>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    if (e != hipSuccess) (void)hipGetLastError();
    state = e == hipSuccess ? 1 : -1;
  }
  return state == 1;
}

// ---------------------------------------------------------------------------
// Slice kernel (at most 64 rows): the skinny kernel's slice sums, left
// unfolded.  A workgroup takes 16 output columns and a few consecutive K
// slices, one per wave, and writes each slice's sums to P [slices][M][N]
// (float); whoever consumes P adds the slices in ascending order, which is
// the order every other kernel uses.  Cutting K over workgroups puts a
// product with few output columns on all CUs (a CU alone streams its weights
// slowly), at the price of the fold, which the consumer (add_rmsnorm_kernel)
// does on the way.
// ---------------------------------------------------------------------------
template <typename T, int MT>
__global__ __launch_bounds__(256) void gemm_slices_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                          float* __restrict__ P, int M, int N, int K, long ldx,
                                                          int kslice, int aligned, int slices_per_group) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int nslices = (K + kslice - 1) / kslice;
  const int s = blockIdx.y * slices_per_group + wave;
  if (wave >= slices_per_group || s >= nslices) return;

  f32x4 acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int k_begin = s * kslice;
  const int k_end = min(K, k_begin + kslice);
  constexpr int UNR = 8;  // a slice of 256 elements in one round of loads
  for (int k0 = k_begin; k0 < k_end; k0 += UNR * A::KCHUNK) {
    vec_t w[UNR], x[MT][UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * A::KCHUNK + g * A::VEC;
      const bool in = k0 + u * A::KCHUNK < k_end;
      w[u] = load_vec<T>(W, n0 + row16, k, K, K, n0 + row16 < N && in, aligned);
#pragma unroll
      for (int j = 0; j < MT; ++j)
        x[j][u] = load_vec<T>(X, j * 16 + row16, k, K, ldx, j * 16 + row16 < M && in, aligned);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (k0 + u * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
      for (int j = 0; j < MT; ++j) A::mma(acc[j], w[u], x[j][u]);
    }
  }
  // lane: rows j * 16 + row16 of X, columns n0 + 4g .. n0 + 4g + 3
  const int n = n0 + g * 4;
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = j * 16 + row16;
    if (m >= M || n >= N) continue;
    float* dst = P + ((long)s * M + m) * N + n;
    if (n + 3 < N && (N & 3) == 0) {
      *reinterpret_cast<f32x4*>(dst) = acc[j];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) dst[r] = acc[j][r];
    }
  }
}

// The slice kernel for an operand that is still the per-split sums of an attention launch (decoded tokens,
// at most 16 rows): X [m][k] is the output of token m, head k / head_dim, column k % head_dim, which the fold
// over the token's `splits` partial results (acc, m, l), ascending from the empty state, skipping empty ones,
// then acc / l rounded to T, would give.  A workgroup takes one K slice and 64 output columns: its four waves
// fold the slice's elements into LDS together first (every group of 64 columns repeats that, which costs
// little while rows times splits are few), then each wave multiplies its 16 columns from there.  The launch
// that would fold them into an output, and the round trip of that output, are saved.  Partial row of (token
// m, head h, split s): (m * heads + h) * splits + s, as the attention kernels lay single decoded tokens out.
// The fold is the attention library's fold_split operation by operation, and the chain of a slice is
// gemm_slices_kernel's: the same bits as fold, then product.
// UNITS, SPLITS: a thread's groups of four elements whose sums are requested together, and the most splits
// each has (instances for few and for more of either; splits <= SPLITS and the host's choice of UNITS
// change nothing in the arithmetic).  REVERSED: a wrong variant for the tests' control library (descending fold).
template <typename T, bool REVERSED, int UNITS, int SPLITS>
__global__ __launch_bounds__(256) void gemm_slices_folded_kernel(const float* __restrict__ part_acc,
                                                                 const float* __restrict__ part_ml, int splits,
                                                                 int head_dim, const T* __restrict__ W,
                                                                 float* __restrict__ P, int M, int N, int K, int kslice) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char folded_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 64 + wave * 16;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int s = blockIdx.y;
  const int k_begin = s * kslice;
  const int k_end = min(K, k_begin + kslice);
  const int row_stride = kslice + 16 / (int)sizeof(T);  // elements; the pad spreads the rows over the banks
  T* xs = reinterpret_cast<T*>(folded_lds);             // [M][row_stride]
  const int heads = K / head_dim;

  // The weights of the slice's first round are requested before the sums: both are on their way together, and
  // the fold runs while the weights arrive.
  constexpr int UNR = 8;  // a slice of 256 elements in one round of loads
  vec_t w_first[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int k = k_begin + u * A::KCHUNK + g * A::VEC;
    w_first[u] = load_vec<T>(W, n0 + row16, k, K, K, n0 + row16 < N && k_begin + u * A::KCHUNK < k_end, true);
  }
  __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move these loads down to their use, behind the fold)

  // A unit is four neighbouring elements of one row; thread t takes the units t, t + 256, ...  A unit's
  // splits are folded one after the other; the sums of UNITS units are requested together.
  const int quads = kslice / 4;
  const int units = M * quads;
  for (int u0 = threadIdx.x; u0 < units; u0 += 256 * UNITS) {
    f32x4 acc[UNITS][SPLITS];
    float2 ml[UNITS][SPLITS];
#pragma unroll
    for (int j = 0; j < UNITS; ++j) {
      const int unit = min(u0 + 256 * j, units - 1);                 // (clamped: loaded, not used)
      const int m = unit / quads;
      const int k = min(k_begin + 4 * (unit - m * quads), K - 4);
      const int head = k / head_dim;
      const long pr0 = ((long)m * heads + head) * splits;
      const float* from = part_acc + (k - head * head_dim);
#pragma unroll
      for (int sp = 0; sp < SPLITS; ++sp) {
        const int at = min(sp, splits - 1);
        const long pr = pr0 + (REVERSED ? splits - 1 - at : at);
        acc[j][sp] = *reinterpret_cast<const f32x4*>(from + pr * head_dim);
        ml[j][sp] = *reinterpret_cast<const float2*>(part_ml + pr * 2);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request is made before the first sum is used
#pragma unroll
    for (int j = 0; j < UNITS; ++j) {
      f32x4 run_acc = f32x4{0.f, 0.f, 0.f, 0.f};
      float run_m = kNegSentinel, run_l = 0.f;
#pragma unroll
      for (int sp = 0; sp < SPLITS; ++sp) {
        if (sp < splits && ml[j][sp].y > 0.f) {  // fold_split on these four columns
          const float m_new = fmaxf(run_m, ml[j][sp].x);
          const float fa = softmax_exp<T>(run_m - m_new);
          const float fb = softmax_exp<T>(ml[j][sp].x - m_new);
#pragma unroll
          for (int e = 0; e < 4; ++e) run_acc[e] = run_acc[e] * fa + acc[j][sp][e] * fb;
          run_l = run_l * fa + ml[j][sp].y * fb;
          run_m = m_new;
        }
      }
      const int unit = u0 + 256 * j;
      const int m = unit / quads;
      const int k = k_begin + 4 * (unit - m * quads);
      if (unit < units && k < k_end) {  // the unit is folded: acc / l, rounded as the attention output is
        T* dst = xs + (long)m * row_stride + (k - k_begin);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[e] = from_f32<T>(run_l > 0.f ? run_acc[e] / run_l : 0.f);
      }
    }
  }
  __syncthreads();
  if (n0 >= N) return;

  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = k_begin; k0 < k_end; k0 += UNR * A::KCHUNK) {
    vec_t w[UNR], x[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * A::KCHUNK + g * A::VEC;
      const bool in = k0 + u * A::KCHUNK < k_end;
      w[u] = k0 == k_begin ? w_first[u] : load_vec<T>(W, n0 + row16, k, K, K, n0 + row16 < N && in, true);
      x[u] = (row16 < M && in && k < k_end) ? *reinterpret_cast<const vec_t*>(xs + (long)row16 * row_stride + (k - k_begin))
                                            : A::zero();
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (k0 + u * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
      A::mma(acc, w[u], x[u]);
    }
  }
  const int n = n0 + g * 4;
  if (row16 < M && n < N) {
    float* dst = P + ((long)s * M + row16) * N + n;
    if (n + 3 < N && (N & 3) == 0) {
      *reinterpret_cast<f32x4*>(dst) = acc;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) dst[r] = acc[r];
    }
  }
}

// The slice kernel for many rows and many columns: a wave takes one K slice of NTL column tiles (16 * NTL
// columns) and all the rows, so a chunk of X that it has loaded meets NTL chunks of weights and a chunk of
// weights MT chunks of X: at 64 rows and 64 columns the rows of X are read once for every byte of weights,
// where the kernel above reads them four times over.  The chain of a slice is the same (ascending chunks,
// from zero), so are the bits.  UNR chunks are loaded at a time, then multiplied; the CU's other waves
// cover the wait.
template <typename T, int MT, int NTL, int UNR>
__global__ __launch_bounds__(256) void gemm_slices_wide_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                               float* __restrict__ P, int M, int N, int K, long ldx,
                                                               int kslice, int aligned, int slices_per_group) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16 * NTL;
  const int s = blockIdx.y * slices_per_group + wave;
  if (wave >= slices_per_group || s >= (K + kslice - 1) / kslice) return;
  const int row16 = lane & 15;
  const int g = lane >> 4;

  f32x4 acc[NTL][MT];
#pragma unroll
  for (int i = 0; i < NTL; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int k_begin = s * kslice;
  const int k_end = min(K, k_begin + kslice);
  for (int k0 = k_begin; k0 < k_end; k0 += UNR * A::KCHUNK) {
    vec_t w[UNR][NTL], x[UNR][MT];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * A::KCHUNK + g * A::VEC;
      const bool in = k0 + u * A::KCHUNK < k_end;
#pragma unroll
      for (int i = 0; i < NTL; ++i) {
        const int n = n0 + i * 16 + row16;
        w[u][i] = load_vec<T>(W, n, k, K, K, n < N && in, aligned);
      }
#pragma unroll
      for (int j = 0; j < MT; ++j)
        x[u][j] = load_vec<T>(X, j * 16 + row16, k, K, ldx, j * 16 + row16 < M && in, aligned);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (k0 + u * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
      for (int i = 0; i < NTL; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j) A::mma(acc[i][j], w[u][i], x[u][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < NTL; ++i) {
    const int n = n0 + i * 16 + g * 4;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int m = j * 16 + row16;
      if (m >= M || n >= N) continue;
      float* dst = P + ((long)s * M + m) * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<f32x4*>(dst) = acc[i][j];
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) dst[r] = acc[i][j][r];
      }
    }
  }
}

// The slice kernel as a walk (products with many K slices and enough column
// blocks that workgroups can take several): wave = slice, its rows of X stay
// in registers, the weights of the next units are in flight across column
// blocks as in the streaming kernel.  The waves share nothing, so there is no
// barrier.
template <typename T, int MT, int XC>
__global__ __launch_bounds__(256) void gemm_slices_stream_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                                 float* __restrict__ P, int M, int N, int K, long ldx,
                                                                 int kslice, int aligned, int slices_per_group,
                                                                 int blocks) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int UC = 4;                          // chunks per unit
  constexpr int UNITS = XC / UC;                 // units per column block
  constexpr int RING = (MT * XC <= 24) ? 4 : 2;  // unit buffers in registers
  constexpr int AHEAD = RING - 1;
  static_assert(XC % UC == 0 && (UNITS % RING == 0 || (2 * UNITS) % RING == 0), "units and ring");
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int nslices = (K + kslice - 1) / kslice;
  const int s = blockIdx.y * slices_per_group + wave;
  if (wave >= slices_per_group || s >= nslices) return;
  const int k_begin = s * kslice;
  const int k_end = min(K, k_begin + kslice);
  const int walkers = gridDim.x;
  const int m_base = blockIdx.z * MT * 16;  // more than 16 * MT rows: groups of rows, each with workgroups of its own

  auto fetch = [&](int b, int q, vec_t (&dst)[UC]) LS_INLINED {
    const int n = b * 16 + row16;
#pragma unroll
    for (int c = 0; c < UC; ++c) {
      const int kc = k_begin + (q * UC + c) * A::KCHUNK;
      dst[c] = load_vec<T>(W, n, kc + g * A::VEC, K, K, n < N && kc < k_end, aligned);
    }
  };
  vec_t wbuf[RING][UC];
  int b = blockIdx.x;
#pragma unroll
  for (int u = 0; u < AHEAD; ++u) {
    const int bu = b + (u / UNITS) * walkers;
    if (bu < blocks) fetch(bu, u % UNITS, wbuf[u % RING]);
  }
  vec_t xs[MT][XC];
#pragma unroll
  for (int j = 0; j < MT; ++j)
#pragma unroll
    for (int c = 0; c < XC; ++c) {
      const int kc = k_begin + c * A::KCHUNK;
      xs[j][c] = load_vec<T>(X, m_base + j * 16 + row16, kc + g * A::VEC, K, ldx,
                             m_base + j * 16 + row16 < M && kc < k_end, aligned);
    }

  auto block_step = [&](auto par) LS_INLINED {
    constexpr int P0 = decltype(par)::value;
    f32x4 acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int idx = 0; idx < UNITS; ++idx) {
      const int far_block = b + ((idx + AHEAD) / UNITS) * walkers;
      if (far_block < blocks) fetch(far_block, (idx + AHEAD) % UNITS, wbuf[(P0 + idx + AHEAD) % RING]);
#pragma unroll
      for (int c = 0; c < UC; ++c) {
        if (k_begin + (idx * UC + c) * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
        for (int j = 0; j < MT; ++j) A::mma(acc[j], wbuf[(P0 + idx) % RING][c], xs[j][idx * UC + c]);
      }
    }
    const int n = b * 16 + g * 4;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int m = m_base + j * 16 + row16;
      if (m >= M || n >= N) continue;
      float* dst = P + ((long)s * M + m) * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<f32x4*>(dst) = acc[j];
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) dst[r] = acc[j][r];
      }
    }
  };
  while (b < blocks) {
    block_step(std::integral_constant<int, 0>{});
    b += walkers;
    if (UNITS % RING != 0) {
      if (b >= blocks) break;
      block_step(std::integral_constant<int, UNITS % RING>{});
      b += walkers;
    }
  }
}

// ---------------------------------------------------------------------------
// Tiled kernel: BM x BN outputs per workgroup, NWM x NWN waves, each
// (BM/NWM) x (BN/NWN).  Both operands go through LDS in stages of 128 bytes
// of K per row, double buffered: while stage i is multiplied, stage i+1 is
// written to the other buffer and the global loads of stage i+2 are in
// flight.  A wave's accumulators (at most 64 x 64 outputs, twice: the slice
// sum and the total) leave room for two waves a SIMD, which is what hides
// the LDS and barrier latency.  Workgroups are numbered so that those that
// share a weight tile run on the same XCD (each XCD has its own L2).
//
// What bounds the kernel is the rate at which a CU gets operand bytes from
// L2 (measured: every tile shape runs at 45 to 48 GB/s a CU), so the bytes a
// workgroup loads per MFMA decide: (BM + BN) / (BM BN).  Hence eight waves
// with 128 x 256 outputs where that many tiles fill the CUs, and the 2 x 2
// grids of waves below that.
// ---------------------------------------------------------------------------
constexpr int kRowBytes = 128;               // bytes of K per row per stage (two chunks)
constexpr int kRowStride = kRowBytes + 16;   // padded LDS row

template <typename T, int EPI, int BM, int BN, int PD, bool AL, int NWM = 2, int NWN = 2>
__global__ __launch_bounds__(64 * NWM * NWN) void gemm_tiled_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                         void* __restrict__ C, int M, int N, int K, long ldx,
                                                         long ldc, int kslice, int vec_ok, int tiles_m, int tiles_n,
                                                         int out_cols) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int BK = kRowBytes / sizeof(T);  // elements of K per stage
  constexpr int TI = BN / (16 * NWN);        // weight tiles (16 columns) per wave
  constexpr int TJ = BM / (16 * NWM);        // row tiles per wave
  constexpr int PASS = 8 * NWM * NWN;        // rows per staging pass: 8 threads a row
  constexpr int WP = BN / PASS;              // staging passes over the weight tile
  constexpr int XP = BM / PASS;
  static_assert(BN % PASS == 0 && BM % PASS == 0 && TI * 16 * NWN == BN && TJ * 16 * NWM == BM, "tile shape");
  constexpr int STAGE_BYTES = (BM + BN) * kRowStride;
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * STAGE_BYTES];

  // XCD-aware numbering: workgroup ids go round the eight XCDs; give each XCD a contiguous run of tiles
  int id = blockIdx.x;
  const int total_tiles = tiles_m * tiles_n;
  if (total_tiles % 8 == 0) id = (id % 8) * (total_tiles / 8) + id / 8;
#if LS_GEMM_GROUP_M > 0
  // ... and inside bands of LS_GEMM_GROUP_M row tiles, so that the workgroups that run together on an XCD
  // form a block of tiles with few distinct operand tiles (those stay in the XCD's L2)
  const int band = id / (LS_GEMM_GROUP_M * tiles_n);
  const int in_band = id % (LS_GEMM_GROUP_M * tiles_n);
  const int band_rows = min(LS_GEMM_GROUP_M, tiles_m - band * LS_GEMM_GROUP_M);
  const int tile_m = band * LS_GEMM_GROUP_M + in_band % band_rows;
  const int tile_n = in_band / band_rows;
#else
  const int tile_m = id % tiles_m;
  const int tile_n = id / tiles_m;
#endif
  const int m_base = tile_m * BM;
  const int n_base = tile_n * BN;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wn = (wave % NWN) * (BN / NWN);
  const int wm = (wave / NWN) * (BM / NWM);
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int st_row = threadIdx.x >> 3;             // staging: 8 threads per row, PASS rows per pass
  const int st_col = (threadIdx.x & 7) * A::VEC;

  f32x4 total[TI][TJ];
  f32x4 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      total[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  // PD stages of global loads are in flight in registers (slot = stage % PD).
  // AL (rows and K 16-byte aligned, K a multiple of VEC): the loads are unconditional, from addresses
  // clamped into the matrix, and nothing reads their registers before the stage is written to LDS, so
  // the loads of PD stages really are in flight together (a zero selected right behind a load makes the
  // compiler wait for it there).  Rows beyond M or N then hold copies of the last row: their products
  // land in outputs that the epilogue does not store.  Only columns from K on must read as zero, and
  // those are cleared on the way to LDS.
  vec_t wv[PD][WP], xv[PD][XP];
  const T* w_src[WP];
  const T* x_src[XP];
  if (AL) {
#pragma unroll
    for (int p = 0; p < WP; ++p) w_src[p] = W + (long)min(n_base + st_row + PASS * p, N - 1) * K;
#pragma unroll
    for (int p = 0; p < XP; ++p) x_src[p] = X + (long)min(m_base + st_row + PASS * p, M - 1) * ldx;
  }
  auto fetch = [&](int slot, int k0) LS_INLINED {
    if (AL) {
      const int k = min(k0 + st_col, K - A::VEC);
#pragma unroll
      for (int p = 0; p < WP; ++p) wv[slot][p] = *reinterpret_cast<const vec_t*>(w_src[p] + k);
#pragma unroll
      for (int p = 0; p < XP; ++p) xv[slot][p] = *reinterpret_cast<const vec_t*>(x_src[p] + k);
      return;
    }
#pragma unroll
    for (int p = 0; p < WP; ++p) {
      const int r = st_row + PASS * p;
      wv[slot][p] = load_vec<T>(W, n_base + r, k0 + st_col, K, K, n_base + r < N, false);
    }
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int r = st_row + PASS * p;
      xv[slot][p] = load_vec<T>(X, m_base + r, k0 + st_col, K, ldx, m_base + r < M, false);
    }
  };
  auto stash = [&](int slot, int buf, int k0) LS_INLINED {
    unsigned char* w_lds = lds + buf * STAGE_BYTES;
    unsigned char* x_lds = w_lds + BN * kRowStride;
#pragma unroll
    for (int p = 0; p < WP; ++p)
      *reinterpret_cast<vec_t*>(&w_lds[(st_row + PASS * p) * kRowStride + st_col * sizeof(T)]) = wv[slot][p];
#pragma unroll
    for (int p = 0; p < XP; ++p)
      *reinterpret_cast<vec_t*>(&x_lds[(st_row + PASS * p) * kRowStride + st_col * sizeof(T)]) = xv[slot][p];
    if (AL && k0 + BK > K) {  // uniform: the last stage where K is no multiple of BK; its columns from K on are cleared
      if (k0 + st_col >= K) {
#pragma unroll
        for (int p = 0; p < WP; ++p)
          *reinterpret_cast<vec_t*>(&w_lds[(st_row + PASS * p) * kRowStride + st_col * sizeof(T)]) = A::zero();
#pragma unroll
        for (int p = 0; p < XP; ++p)
          *reinterpret_cast<vec_t*>(&x_lds[(st_row + PASS * p) * kRowStride + st_col * sizeof(T)]) = A::zero();
      }
    }
  };

  // the stages of this workgroup: all of K, or (kSliceSums) those of its group of slices
  constexpr bool SLICES = EPI == kSliceSums;
  const int all_stages = (K + BK - 1) / BK;
  const int first_stage = SLICES ? (int)blockIdx.y * out_cols * (kslice / BK) : 0;
  const int stages = SLICES ? min(all_stages - first_stage, out_cols * (kslice / BK)) : all_stages;
  auto k_of = [&](int st) LS_INLINED { return (first_stage + st) * BK; };
  auto store_slice = [&](int slice) LS_INLINED {  // the sums of one slice to their place among the slice sums
    float* sums = reinterpret_cast<float*>(C) + (long)slice * M * N;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        float t[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        epilogue4<T, kStoreF32>(sums, ldc, m_base + wm + j * 16 + row16, n_base + wn + i * 16 + g * 4, M, N, t, vec_ok);
      }
  };
  // stage s lives in register slot s % PD until it is written to LDS buffer s % 2
  fetch(0, k_of(0));
  stash(0, 0, k_of(0));
  // (AL: stages past the end are fetched too, from clamped addresses: with no condition around a
  // fetch the compiler can count which loads are still in flight when a stage goes to LDS)
#pragma unroll
  for (int u = 1; u <= PD; ++u)
    if (AL || u < stages) fetch(u % PD, k_of(u));
  for (int base = 0; base < stages; base += PD) {
#pragma unroll
    for (int u = 0; u < PD; ++u) {  // unrolled so that the register slots are static
      const int st = base + u;
      if (st >= stages) break;
      const int k0 = k_of(st);
      if (st > 0 && k0 % kslice == 0) {  // a stage never straddles a slice: kslice is a multiple of BK
        if (SLICES) store_slice(k0 / kslice - 1);
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
          for (int j = 0; j < TJ; ++j) {
#pragma unroll
            for (int r = 0; r < 4; ++r) total[i][j][r] = total[i][j][r] + acc[i][j][r];
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
      }
      __syncthreads();  // stage st is in its buffer; the other buffer has been read by every wave
      if (AL || st + 1 < stages) {  // (AL: past the last stage too, into the buffer that nobody reads any more)
        stash((u + 1) % PD, (st + 1) & 1, k_of(st + 1));
        if (AL || st + 1 + PD < stages) fetch((u + 1) % PD, k_of(st + 1 + PD));
      }
      const unsigned char* w_lds = lds + (st & 1) * STAGE_BYTES;
      const unsigned char* x_lds = w_lds + BN * kRowStride;
      // the fragments of the second chunk are read while the first is multiplied
      vec_t a[2][TI], b[2][TJ];
      auto fragments = [&](int c) LS_INLINED {
#pragma unroll
        for (int i = 0; i < TI; ++i)
          a[c][i] = *reinterpret_cast<const vec_t*>(&w_lds[(wn + i * 16 + row16) * kRowStride + c * 64 + g * 16]);
#pragma unroll
        for (int j = 0; j < TJ; ++j)
          b[c][j] = *reinterpret_cast<const vec_t*>(&x_lds[(wm + j * 16 + row16) * kRowStride + c * 64 + g * 16]);
      };
      fragments(0);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        // The skinny kernel visits a chunk iff it starts below K; do the same.
        if (k0 + c * A::KCHUNK >= K) break;
        if (c == 0 && LS_GEMM_READ_AHEAD) fragments(1);
        if (c == 1 && !LS_GEMM_READ_AHEAD) fragments(1);
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
          for (int j = 0; j < TJ; ++j) A::mma(acc[i][j], a[c][i], b[c][j]);
      }
    }
  }
  if constexpr (SLICES) {
    if (stages > 0) store_slice(k_of(stages - 1) / kslice);
  } else {
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) total[i][j][r] = total[i][j][r] + acc[i][j][r];

    if (EPI == kSwiGLU) {
      // the wave's weight tiles come in pairs (gate t, up t)
#pragma unroll
      for (int i = 0; i < TI; i += 2)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
          float gate[4] = {total[i][j][0], total[i][j][1], total[i][j][2], total[i][j][3]};
          float up[4] = {total[i + 1][j][0], total[i + 1][j][1], total[i + 1][j][2], total[i + 1][j][3]};
          epilogue_swiglu4<T>(C, ldc, m_base + wm + j * 16 + row16, (n_base + wn + i * 16) / 2 + g * 4, M, out_cols,
                              gate, up, vec_ok);
        }
      return;
    }
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        float t[4] = {total[i][j][0], total[i][j][1], total[i][j][2], total[i][j][3]};
        epilogue4<T, EPI>(C, ldc, m_base + wm + j * 16 + row16, n_base + wn + i * 16 + g * 4, M, N, t, vec_ok);
      }
  }
}

template <typename T, int EPI>
int launch_gemm(const void* X, const void* W, void* C, int M, int N, int K, long ldx, long ldc, const float* norm_w,
                float eps, int out_cols, hipStream_t stream) {
  int kslice = kslice_for(K);
  if (LS_MUTANT_HOST(kMutantKsliceByRows) && M > 16 && M <= 64) kslice *= 2;  // the mutant: K blocking that depends on the rows of the launch
  const int nslices = (K + kslice - 1) / kslice;
  constexpr int VEC = Atom<T>::VEC;
  constexpr int NT = (EPI == kSwiGLU) ? 2 : 1;
  const int aligned = (K % VEC == 0) && (norm_w || ldx % VEC == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(W) % 16 == 0);
  const size_t out_size = (EPI == kStore || EPI == kSwiGLU) ? sizeof(T) : sizeof(float);
  const int vec_ok = (ldc % 4 == 0) && (reinterpret_cast<uintptr_t>(C) % (4 * out_size) == 0);
  const T* w = reinterpret_cast<const T*>(W);
  if (norm_w && M > 16) return fail("gemm: the fused norm prologue takes at most 16 rows, got %d", M);
  // Up to 64 rows the skinny kernel; but with more than 16 rows and very many columns (the logits
  // head) its workgroups re-read all rows of X for 16 columns each, and the tiled kernel reads less.
  const int mt_rows = (M + 15) / 16;
  const int col_blocks = (N + 16 * NT - 1) / (16 * NT);
  // With more than 16 rows the tiled kernel does better wherever it has a workgroup for every CU (its
  // workgroups read the rows of X once for 64 columns, through LDS, and 64 columns of weights a workgroup
  // keep enough loads in flight): from 33 rows on always (Qwen3-8B sizes, gate and up at 64 rows: 85 -> 50
  // us), from 17 rows on for SwiGLU, where the streaming kernel has two weight tiles a column block and
  // holds less in flight (58 -> 46 us at 32 rows; the logits head at 24 rows: streaming 257, tiled 307 us).
  const bool tiled_fills = !norm_w && M <= 64 && (N + 63) / 64 >= compute_units() &&
                           (M > 32 || (M > 16 && EPI == kSwiGLU));
  const int xc = kslice / Atom<T>::KCHUNK;  // chunks per slice
  // The streaming kernel where a workgroup would get more than one column block: a CU holds 16 waves
  // of it (one per K slice), so 16 / nslices workgroups.
  const int stream_wgs = compute_units() * (16 / nslices > 0 ? 16 / nslices : 1);
  // up to 32 rows one group of rows; up to 64 two groups of 32 that share the weights through L2
  const int row_groups = mt_rows <= 2 ? 1 : 2;
  const int group_tiles = mt_rows <= 2 ? mt_rows : 2;
  const size_t stream_lds = 2 * (size_t)nslices * NT * group_tiles * 256 * sizeof(float);  // two sets of slice sums
  // (two groups read the weights twice, the second time rarely from L2 in practice: with very many
  // columns, where the tiled kernel does well, they are not worth it)
  // (with fewer than eight slices the skinny kernel's small workgroups, several a CU, do as well or better)
  if (!norm_w && mt_rows <= 4 && !tiled_fills && xc % 4 == 0 && xc * group_tiles <= 16 && nslices >= 8 && nslices <= 16 &&
      col_blocks * row_groups > stream_wgs && stream_lds <= 128 * 1024 && !(row_groups > 1 && N >= 32768) &&
      LS_GEMM_STREAM) {
    int walkers = stream_wgs / row_groups;
    const int rounds = (col_blocks + walkers - 1) / walkers;
    walkers = (col_blocks + rounds - 1) / rounds;
    if (row_groups > 1) walkers = (walkers + 7) / 8 * 8;  // whole rounds of the XCDs, see the kernel
    dim3 grid(walkers * row_groups);
    bool launched = true;
#define LS_STREAM(MT_, XC_)                                                                                       \
  if (stream_lds_ready<T, MT_, EPI, XC_>(stream_lds))                                                             \
    hipLaunchKernelGGL((gemm_stream_kernel<T, MT_, EPI, XC_>), grid, dim3(nslices * 64), stream_lds, stream,      \
                       reinterpret_cast<const T*>(X), w, C, M, N, K, ldx, ldc, kslice, aligned, vec_ok, out_cols, \
                       col_blocks, row_groups);                                                                   \
  else                                                                                                            \
    launched = false
    if (group_tiles == 1 && xc == 8) LS_STREAM(1, 8);
    else if (group_tiles == 1 && xc == 16) LS_STREAM(1, 16);
    else if (group_tiles == 2 && xc == 8) LS_STREAM(2, 8);
    else launched = false;
#undef LS_STREAM
    if (launched) return check_launch("gemm");
  }
  // 32 to 64 rows over a product that neither fills the CUs with 64-column tiles nor has a streaming kernel
  // for its slice length (QKV of Qwen3-14B and 32B sizes: slices of 512): the skinny kernel re-reads all
  // rows of X for 16 columns a workgroup; tiles of 64 x 32 outputs where they give most CUs a workgroup
  // (measured at 64 rows: N = 10,240, K = 5,120 83 -> 49 us; N = 7,168 56 -> 35 us; at 17 rows no gain).
  if constexpr (EPI != kSwiGLU) {
    if (LS_GEMM_NARROW && !norm_w && aligned && M >= 32 && M <= 64 && !tiled_fills && N < 32768 &&
        (N + 31) / 32 >= compute_units() * 7 / 10) {
      const int tiles_n = (N + 31) / 32;
      hipLaunchKernelGGL((gemm_tiled_kernel<T, EPI, 64, 32, LS_GEMM_PD_SMALL, true, 2, 2>), dim3(tiles_n), dim3(256), 0,
                         stream, reinterpret_cast<const T*>(X), w, C, M, N, K, ldx, ldc, kslice, vec_ok, 1, tiles_n,
                         out_cols);
      return check_launch("gemm");
    }
  }
  if (M <= 64 && !tiled_fills && !(M > 16 && N >= 32768)) {
    const int mt = (M + 15) / 16;
    // 16 waves leave 128 registers a lane: only for one or two row tiles
    const int nw = (nslices > 8 && mt * NT <= 2) ? 16 : (nslices > 4 ? 8 : 4);
    dim3 grid((N + 16 * NT - 1) / (16 * NT));
    const size_t lds = ((size_t)nslices * NT * mt * 256 + (norm_w ? 80 : 0)) * sizeof(float);
#define LS_SKINNY(MT_, NW_, NORM_)                                                                              \
  hipLaunchKernelGGL((gemm_skinny_kernel<T, MT_, NW_, EPI, NORM_>), grid, dim3(NW_ * 64), lds, stream, X, w, C, M, N, \
                     K, ldx, ldc, kslice, aligned, vec_ok, norm_w, eps, out_cols)
    if (norm_w) {
      if (nw >= 8) LS_SKINNY(1, 8, true); else LS_SKINNY(1, 4, true);
    } else if (nw == 16) {
      if (mt == 1) LS_SKINNY(1, 16, false); else LS_SKINNY(2, 16, false);
    } else if (nw == 8) {
      if (mt == 1) LS_SKINNY(1, 8, false); else if (mt == 2) LS_SKINNY(2, 8, false);
      else if (mt == 3) LS_SKINNY(3, 8, false); else LS_SKINNY(4, 8, false);
    } else {
      if (mt == 1) LS_SKINNY(1, 4, false); else if (mt == 2) LS_SKINNY(2, 4, false);
      else if (mt == 3) LS_SKINNY(3, 4, false); else LS_SKINNY(4, 4, false);
    }
#undef LS_SKINNY
  } else {
    // Large products take 128 x 128 tiles (least LDS traffic per MFMA); smaller ones take
    // 64 x 64 tiles so that every CU has several workgroups, with a deeper register prefetch.
    const long big_tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
#define LS_TILED_WAVES(BM_, BN_, PD_, AL_, NWM_, NWN_)                                                         \
  {                                                                                                             \
    const int tiles_m = (M + BM_ - 1) / BM_, tiles_n = (N + BN_ - 1) / BN_;                                       \
    hipLaunchKernelGGL((gemm_tiled_kernel<T, EPI, BM_, BN_, PD_, AL_, NWM_, NWN_>), dim3(tiles_m * tiles_n),      \
                       dim3(64 * NWM_ * NWN_), 0, stream, reinterpret_cast<const T*>(X), w, C, M, N, K, ldx, ldc, \
                       kslice, vec_ok, tiles_m, tiles_n, out_cols);                                             \
  }
#define LS_TILED(BM_, BN_, PD_, AL_) LS_TILED_WAVES(BM_, BN_, PD_, AL_, 2, 2)
    // 128 x 256 tiles load a quarter fewer operand bytes per MFMA (measured at 2,048 rows: gate and up of
    // Qwen3-8B sizes 511 -> 446 us, down 246 -> 211 us), but a CU holds one such workgroup, so a last
    // round that leaves CUs idle costs more than it does with the smaller tiles, two of which share a CU
    const long wide_tiles = (long)((M + 127) / 128) * ((N + 255) / 256);
    const long cus = compute_units();
    const long wide_rounds = (wide_tiles + cus - 1) / cus;
    const bool wide_fills = LS_GEMM_WIDE && sizeof(T) == 2 && M > LS_GEMM_BIG_ROWS && wide_tiles >= cus &&
                            (wide_rounds >= 8 || wide_tiles * 100 >= wide_rounds * cus * LS_GEMM_WIDE_FILL);
    // (operands that are not 16-byte aligned take the small tiles, element by element: every tile
    // shape gives the same bits)
    if (!aligned) LS_TILED(64, 64, LS_GEMM_PD_SMALL, false)
    else if (wide_fills) {
      if constexpr (sizeof(T) == 2) LS_TILED_WAVES(128, 256, LS_GEMM_PD_WIDE, true, 2, 4)
    }
    else if (big_tiles >= (LS_GEMM_BIG ? LS_GEMM_BIG : cus) && M > LS_GEMM_BIG_ROWS) LS_TILED(128, 128, LS_GEMM_PD_BIG, true)
    // up to 64 rows over so many columns that tiles of 128 columns still give every CU a workgroup (the
    // logits head, gate and up of 32B sizes): every workgroup reads all rows of X, so half as many
    // workgroups halve that traffic (gate and up of 32B sizes at 64 rows 135 -> 112 us, the head 82 -> 77 us)
    else if (LS_GEMM_ROWS64_WIDE && M <= 64 && (N + 127) / 128 >= cus)
      LS_TILED_WAVES(64, 128, LS_GEMM_PD_SMALL, true, 2, 4)
    else LS_TILED(64, 64, LS_GEMM_PD_SMALL, true)
#undef LS_TILED
#undef LS_TILED_WAVES
  }
  return check_launch("gemm");
}

}  // namespace ls

// dtype: 0 float32, 1 bfloat16.  epilogue: 0 store in dtype, 1 store float,
// 2 add to float, 3 SwiGLU of interleaved gate/up tiles (N = rows of W, the
// output has out_cols <= N/2 columns; rows of W beyond them are padding).  X [M,K] with ldx elements per row, W [N,K]
// contiguous, C with ldc elements per row.  With norm_w (float [K]) X is the
// float residual stream and is RMS-normalised on the fly (M <= 16).
extern "C" int ls_gemm(int dtype, int epilogue, const void* X, const void* W, void* C, int M, int N, int K, long ldx,
                       long ldc, const float* norm_w, float eps, int out_cols, void* stream) {
  using namespace ls;
  LS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: sizes must be positive, got M=%d N=%d K=%d", M, N, K);
  if (epilogue != kSwiGLU) out_cols = N;
  LS_REQUIRE(out_cols > 0 && (epilogue != kSwiGLU || (out_cols <= N / 2 && out_cols > N / 2 - 16)),
             "gemm: %d output columns do not fit %d interleaved weight rows", out_cols, N);
  LS_REQUIRE(ldx >= K && ldc >= out_cols, "gemm: row strides ldx=%ld ldc=%ld are shorter than K=%d / %d columns", ldx,
             ldc, K, out_cols);
  LS_REQUIRE(epilogue != kSwiGLU || N % 32 == 0, "gemm: the SwiGLU epilogue needs interleaved tiles, N=%d", N);
  LS_REQUIRE(X && W && C, "gemm: null operand");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define LS_GEMM_CASE(T_)                                                                              \
  switch (epilogue) {                                                                                 \
    case kStore: return launch_gemm<T_, kStore>(X, W, C, M, N, K, ldx, ldc, norm_w, eps, out_cols, s);          \
    case kStoreF32: return launch_gemm<T_, kStoreF32>(X, W, C, M, N, K, ldx, ldc, norm_w, eps, out_cols, s);    \
    case kAddF32: return launch_gemm<T_, kAddF32>(X, W, C, M, N, K, ldx, ldc, norm_w, eps, out_cols, s);        \
    case kSwiGLU: return launch_gemm<T_, kSwiGLU>(X, W, C, M, N, K, ldx, ldc, norm_w, eps, out_cols, s);        \
    default: return fail("gemm: unknown epilogue %d", epilogue);                                      \
  }
  if (dtype == kF32) { LS_GEMM_CASE(float) }
  if (dtype == kBF16) { LS_GEMM_CASE(bf16_t) }
#undef LS_GEMM_CASE
  return fail("gemm: unknown dtype %d", dtype);
}

extern "C" int ls_gemm_kslice(int K) { return ls::kslice_for(K); }

// Number of K slices of a product over K (the first dimension of the partial sums of ls_gemm_slices).
extern "C" int ls_gemm_slices_count(int K) {
  const int kslice = ls::kslice_for(K);
  return (K + kslice - 1) / kslice;
}

// Rows that ls_gemm_slices takes for a product over K: 64 always; 256 where the kernel that keeps
// its rows of X in registers has an instance for the slice length (more rows are further groups of
// workgroups that walk the same weights).
extern "C" int ls_gemm_slices_max_rows(int dtype, int K) {
  const int xc = ls::kslice_for(K) / (dtype == ls::kF32 ? 16 : 32);
  return (LS_GEMM_STREAM && (xc == 8 || xc == 16)) ? 256 : 64;
}

// Slice sums of X [M,K] @ W [N,K]^T for M <= ls_gemm_slices_max_rows: P [slices][M][N] float, P[s] = the
// sum over K slice s.  The product is P[0] + P[1] + ... added in this order, starting from +0.
extern "C" int ls_gemm_slices(int dtype, const void* X, const void* W, float* P, int M, int N, int K, long ldx,
                              void* stream) {
  using namespace ls;
  LS_REQUIRE(M > 0 && M <= ls_gemm_slices_max_rows(dtype, K) && N > 0 && K > 0,
             "gemm_slices: takes 1 to %d rows with K=%d, got M=%d N=%d", ls_gemm_slices_max_rows(dtype, K), K, M, N);
  LS_REQUIRE(ldx >= K && X && W && P, "gemm_slices: bad operands");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(P) % 16 == 0, "gemm_slices: the partial sums must be 16-byte aligned");
  const int kslice = kslice_for(K);
  const int nslices = (K + kslice - 1) / kslice;
  const int col_blocks = (N + 15) / 16;
  // enough groups of slices to fill the GPU, at most four slices (waves) a workgroup
  int groups = (compute_units() + col_blocks - 1) / col_blocks;
  if (groups > nslices) groups = nslices;
  if (groups < (nslices + 3) / 4) groups = (nslices + 3) / 4;
  const int per_group = (nslices + groups - 1) / groups;
  groups = (nslices + per_group - 1) / per_group;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid(col_blocks, groups);
  const int vec = dtype == kF32 ? 4 : 8;
  const int aligned = (K % vec == 0) && (ldx % vec == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(W) % 16 == 0);
  const int mt = (M + 15) / 16;
  // With more than 16 rows, where the rows of X outweigh the weights of a column block, and at least four
  // workgroups a CU, workgroups walk two or more column blocks each with X in registers (the walk keeps
  // two workgroups a CU).  Up to 16 rows the walk measured no faster: fewer waves, less in flight.
  const int xc = kslice / (dtype == kF32 ? 16 : 32);  // 64-byte chunks per slice
  // row tiles a workgroup holds in registers (xs: 4 * xc registers a tile); more rows go to further groups
  // (24 chunks a slice with two tiles need 268 registers: one wave a SIMD, measured slower than the plain kernel)
  const int group_tiles = xc <= 8 ? std::min(mt, 4) : (xc <= 16 ? std::min(mt, 2) : 0);
  const int row_groups = group_tiles > 0 ? (mt + group_tiles - 1) / group_tiles : 0;
  int rounds =
      (int)std::min<long>(4, (long)col_blocks * groups * std::max(row_groups, 1) / (2L * compute_units()));
  if (mt > 4 && rounds < 1) rounds = 1;  // more than 64 rows: this kernel only, if with one column block a workgroup
  // Enough rows over weights large enough that 64 x 64 tiles times groups of slices give every CU a
  // workgroup: the tiled kernel, which stages both operands in LDS four stages ahead and so keeps twice the
  // bytes of the wide kernel in flight (measured at 64 rows, Qwen3-8B and 32B sizes: O 18.3 -> 12.4 and
  // 44.9 -> 27.8 us, down 42.3 -> 30.3 and 119.9 -> 68.0 us; at 256 rows O 44.5 -> 30.4 and 147.9 -> 68.1 us).
  // A workgroup takes as many slices as give it eight stages, fewer where that leaves CUs without one.
  // From 17 rows on in bfloat16 (from 8 over weights of 64 MB and more, where the kernels of a wave a slice
  // fall to 3.7 TB/s and this one holds 4.2 to 4.6; below that and over smaller weights those are ahead),
  // from 33 rows on in float32.
  const long weight_bytes = (long)N * K * (dtype == kF32 ? 4 : 2);
  const int tiled_from = dtype == kF32 ? 33 : (weight_bytes >= (64L << 20) ? 8 : 17);
  if (LS_GEMM_SLICES_TILED && aligned && M >= tiled_from && N % 4 == 0) {
    const int stages_a_slice = kslice / (128 / (dtype == kF32 ? 4 : 2));
    int per = std::min(nslices, std::max(1, (8 + stages_a_slice - 1) / stages_a_slice));
    const int tiles_m = (M + 63) / 64, tiles_n = (N + 63) / 64;
    auto workgroups = [&](int p) LS_INLINED { return (long)tiles_m * tiles_n * ((nslices + p - 1) / p); };
    while (per > 1 && workgroups(per) < compute_units()) per = (per + 1) / 2;
    if (workgroups(per) >= compute_units()) {
      const int groups_y = (nslices + per - 1) / per;
      dim3 tiled_grid(tiles_m * tiles_n, groups_y);
#define LS_TILED_SLICES(T_)                                                                                          \
  hipLaunchKernelGGL((gemm_tiled_kernel<T_, kSliceSums, 64, 64, LS_GEMM_PD_SMALL, true, 2, 2>), tiled_grid, dim3(256), \
                     0, s, (const T_*)X, (const T_*)W, (void*)P, M, N, K, ldx, (long)N, kslice, 1, tiles_m, tiles_n, per)
      if (dtype == kF32) { LS_TILED_SLICES(float); } else if (dtype == kBF16) { LS_TILED_SLICES(bf16_t); } else return fail("gemm_slices: unknown dtype %d", dtype);
#undef LS_TILED_SLICES
      return check_launch("gemm_slices");
    }
  }
  // More than 16 rows and enough columns that workgroups of 64 columns fill the GPU: the wide kernel.
  {
    const int wide_blocks = (N + 63) / 64;
    const int wide_per_group = std::min(4, nslices);
    const int wide_groups = (nslices + wide_per_group - 1) / wide_per_group;
    if (mt >= 2 && mt <= 4 && (long)wide_blocks * wide_groups >= LS_GEMM_SLICES_WIDE_WGS && xc % LS_GEMM_SLICES_WIDE_UNR == 0 &&
        LS_GEMM_SLICES_WIDE) {
      dim3 wide_grid(wide_blocks, wide_groups);
#define LS_WIDE(T_, MT_)                                                                                          \
  hipLaunchKernelGGL((gemm_slices_wide_kernel<T_, MT_, 4, LS_GEMM_SLICES_WIDE_UNR>), wide_grid,                 \
                     dim3(64 * wide_per_group), 0, s, (const T_*)X, (const T_*)W, P, M, N, K, ldx, kslice, aligned, \
                     wide_per_group)
#define LS_WIDE_MT(T_)                                       \
  if (mt == 2) LS_WIDE(T_, 2); else if (mt == 3) LS_WIDE(T_, 3); else LS_WIDE(T_, 4)
      if (dtype == kF32) { LS_WIDE_MT(float); } else if (dtype == kBF16) { LS_WIDE_MT(bf16_t); } else return fail("gemm_slices: unknown dtype %d", dtype);
#undef LS_WIDE_MT
#undef LS_WIDE
      return check_launch("gemm_slices");
    }
  }
  if ((rounds >= 2 || mt > 4) && mt >= 2 && group_tiles > 0 && xc % 4 == 0 && LS_GEMM_STREAM) {
    int walkers = (col_blocks + rounds - 1) / rounds;
    if (row_groups > 1) walkers = (walkers + 7) / 8 * 8;  // the groups' workgroups of a walk sit on the same XCD
    dim3 walk_grid(walkers, groups, row_groups);
    bool launched = true;
#define LS_WALK(T_, MT_, XC_)                                                                                     \
  hipLaunchKernelGGL((gemm_slices_stream_kernel<T_, MT_, XC_>), walk_grid, dim3(64 * per_group), 0, s, (const T_*)X, \
                     (const T_*)W, P, M, N, K, ldx, kslice, aligned, per_group, col_blocks)
#define LS_WALK_T(T_)                                                          \
  if (group_tiles == 2 && xc == 8) LS_WALK(T_, 2, 8);                          \
  else if (group_tiles == 3 && xc == 8) LS_WALK(T_, 3, 8);                     \
  else if (group_tiles == 4 && xc == 8) LS_WALK(T_, 4, 8);                     \
  else if (group_tiles == 2 && xc == 16) LS_WALK(T_, 2, 16);                   \
  else launched = false
    if (dtype == kF32) { LS_WALK_T(float); } else if (dtype == kBF16) { LS_WALK_T(bf16_t); } else launched = false;
#undef LS_WALK_T
#undef LS_WALK
    if (launched) return check_launch("gemm_slices");
  }
  LS_REQUIRE(mt <= 4, "gemm_slices: no kernel for %d rows with K=%d", M, K);
#define LS_SLICES(T_, MT_)                                                                                       \
  hipLaunchKernelGGL((gemm_slices_kernel<T_, MT_>), grid, dim3(64 * per_group), 0, s, (const T_*)X, (const T_*)W, P, M, \
                     N, K, ldx, kslice, aligned, per_group)
#define LS_SLICES_MT(T_)                                              \
  if (mt == 1) LS_SLICES(T_, 1); else if (mt == 2) LS_SLICES(T_, 2); \
  else if (mt == 3) LS_SLICES(T_, 3); else LS_SLICES(T_, 4)
  if (dtype == kF32) {
    LS_SLICES_MT(float);
  } else if (dtype == kBF16) {
    LS_SLICES_MT(bf16_t);
  } else {
    return fail("gemm_slices: unknown dtype %d", dtype);
  }
#undef LS_SLICES_MT
#undef LS_SLICES
  return check_launch("gemm_slices");
}

// Whether ls_gemm_slices_folded takes this product: at most 16 rows, whole heads of a size that is a
// multiple of four, K a multiple of the load width, at most 32 splits, the folded rows of a slice within
// 64 KB of LDS -- and the plain slice kernel is what ls_gemm_slices itself would run for these sizes (over
// large weights it prefers the tiled kernel from eight rows on, which reads its operand from memory).
extern "C" int ls_gemm_slices_folded_ok(int dtype, int M, int N, int K, int head_dim, int splits) {
  using namespace ls;
  if (dtype != kF32 && dtype != kBF16) return 0;
  if (M < 1 || M > 16 || N < 1 || K < 1 || head_dim < 4 || head_dim % 4 || K % head_dim) return 0;
  if (splits < 1 || splits > 32 || K % (dtype == kF32 ? 4 : 8)) return 0;
  const long weight_bytes = (long)N * K * (dtype == kF32 ? 4 : 2);
  const int tiled_from = dtype == kF32 ? 33 : (weight_bytes >= (64L << 20) ? 8 : 17);
  if (LS_GEMM_SLICES_TILED && M >= tiled_from && N % 4 == 0) return 0;
  const size_t element = dtype == kF32 ? 4 : 2;
  return (size_t)M * (kslice_for(K) + 16 / element) * element <= 64 * 1024;
}

// ls_gemm_slices for an operand that is still `splits` per-split sums a (token, head) of an attention
// launch over single decoded tokens (see gemm_slices_folded_kernel): part_acc [(M * heads) * splits][head_dim],
// part_ml [(M * heads) * splits][2], heads = K / head_dim.  P as ls_gemm_slices leaves it, bit for bit what
// it leaves for the folded and rounded operand.
extern "C" int ls_gemm_slices_folded(int dtype, const float* part_acc, const float* part_ml, int splits, int head_dim,
                                     const void* W, float* P, int M, int N, int K, void* stream) {
  using namespace ls;
  LS_REQUIRE(ls_gemm_slices_folded_ok(dtype, M, N, K, head_dim, splits),
             "gemm_slices_folded: not for M=%d N=%d K=%d head_dim=%d splits=%d (see ls_gemm_slices_folded_ok)", M, N, K,
             head_dim, splits);
  LS_REQUIRE(part_acc && part_ml && W && P, "gemm_slices_folded: null operand");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(P) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(part_acc) % 16 == 0 && reinterpret_cast<uintptr_t>(part_ml) % 8 == 0,
             "gemm_slices_folded: operands must be 16-byte aligned");
  const int kslice = kslice_for(K);
  const int nslices = (K + kslice - 1) / kslice;
  const size_t element = dtype == kF32 ? 4 : 2;
  const size_t lds = (size_t)M * (kslice + 16 / element) * element;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((N + 63) / 64, nslices);
#define LS_FOLDED_N(T_, REV_, UNITS_, SPLITS_)                                                                       \
  hipLaunchKernelGGL((gemm_slices_folded_kernel<T_, REV_, UNITS_, SPLITS_>), grid, dim3(256), lds, s, part_acc, part_ml, \
                     splits, head_dim, (const T_*)W, P, M, N, K, kslice)
  // units of a thread whose sums are in flight together: all of them up to four
  const int mine = (M * (kslice / 4) + 255) / 256;
#define LS_FOLDED_S(T_, REV_, SPLITS_)                       \
  if (mine <= 1) LS_FOLDED_N(T_, REV_, 1, SPLITS_);          \
  else if (mine <= 2) LS_FOLDED_N(T_, REV_, 2, SPLITS_);     \
  else LS_FOLDED_N(T_, REV_, 4, SPLITS_)
#define LS_FOLDED(T_, REV_)                                  \
  if (splits <= 4) { LS_FOLDED_S(T_, REV_, 4); }             \
  else if (splits <= 8) { LS_FOLDED_S(T_, REV_, 8); }        \
  else LS_FOLDED_N(T_, REV_, 1, 32)
#ifdef LS_MUTANTS
  if (LS_MUTANT_HOST(kMutantReversedFoldInProduct)) {
    if (dtype == kF32) { LS_FOLDED(float, true); } else { LS_FOLDED(bf16_t, true); }
    return check_launch("gemm_slices_folded");
  }
#endif
  if (dtype == kF32) { LS_FOLDED(float, false); } else { LS_FOLDED(bf16_t, false); }
#undef LS_FOLDED_S
#undef LS_FOLDED_N
#undef LS_FOLDED
  return check_launch("gemm_slices_folded");
}
