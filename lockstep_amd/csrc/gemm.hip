// C[M,N] = X[M,K] * W[N,K]^T with a fixed summation order per output element.
//
// The order, for every (m, n), whatever M is and whichever kernel runs:
//   K is cut into slices of `kslice` elements (a function of K alone);
//   inside a slice the products are accumulated by a chain of MFMA atoms over
//   ascending 64-byte chunks of K, starting from zero;
//   the slice sums are added in ascending order to a total that starts at +0.
// The skinny kernel (M <= 64, decode) gives each slice to a wave, so the
// weights stream from HBM with many waves in flight; the tiled kernel
// (prefill) walks the slices one after the other with both operands staged
// in LDS.  Both produce the same bits for a row, so a token's projections do
// not depend on how many tokens share its step.
//
// The MFMA runs "swapped": W rows are the first operand, X rows the second,
// so a lane ends with four consecutive n of one row m and stores them as one
// vector.

#include "common.h"

namespace ls {

enum Epilogue : int {
  kStore = 0,     // C[m][n] = total, in the compute dtype
  kStoreF32 = 1,  // C[m][n] = total, float
  kAddF32 = 2,    // C[m][n] += total, float (residual stream)
};

__host__ __device__ inline int kslice_for(int K) { return 256 * ((K + 4095) / 4096); }

template <typename T, int EPI>
__device__ __forceinline__ void epilogue4(void* __restrict__ C, long ldc, int m, int n, int M, int N,
                                          const float total[4], bool vec_ok) {
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
        f32x4 old = *p;
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

// ---------------------------------------------------------------------------
// Skinny kernel: one workgroup per 16 output columns, NW waves, wave w takes
// slices w, w + NW, ...; slice sums meet in LDS and are folded in ascending
// order by the thread that owns the output element.
// ---------------------------------------------------------------------------
template <typename T, int MT, int NW, int EPI>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                               void* __restrict__ C, int M, int N, int K, long ldx,
                                                               long ldc, int kslice, int aligned, int vec_ok) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  extern __shared__ float part[];  // [nslices][MT][256]

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int nslices = (K + kslice - 1) / kslice;
  const int n = n0 + row16;
  const bool n_ok = n < N;

  for (int s = wave; s < nslices; s += NW) {
    f32x4 acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int k_begin = s * kslice;
    const int k_end = min(K, k_begin + kslice);
    // Four chunks at a time: all their loads are issued before the first
    // MFMA needs one, so a wave keeps several kilobytes in flight.
    for (int k0 = k_begin; k0 < k_end; k0 += 4 * A::KCHUNK) {
      vec_t w[4], x[MT][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + u * A::KCHUNK + g * A::VEC;
        const bool in = k0 + u * A::KCHUNK < k_end;
        w[u] = load_vec<T>(W, n, k, K, K, n_ok && in, aligned);
#pragma unroll
        for (int j = 0; j < MT; ++j) x[j][u] = load_vec<T>(X, j * 16 + row16, k, K, ldx, j * 16 + row16 < M && in, aligned);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (k0 + u * A::KCHUNK >= k_end) break;  // uniform: a chunk is visited iff it starts inside the slice
#pragma unroll
        for (int j = 0; j < MT; ++j) A::mma(acc[j], w[u], x[j][u]);
      }
    }
#pragma unroll
    for (int j = 0; j < MT; ++j)
      *reinterpret_cast<f32x4*>(&part[((s * MT + j) * 64 + lane) * 4]) = acc[j];
  }
  __syncthreads();

  for (int idx = threadIdx.x; idx < MT * 64; idx += NW * 64) {
    const int j = idx >> 6;
    const int l = idx & 63;
    float total[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nslices; ++s) {
      f32x4 p = *reinterpret_cast<const f32x4*>(&part[((s * MT + j) * 64 + l) * 4]);
#pragma unroll
      for (int r = 0; r < 4; ++r) total[r] = total[r] + p[r];
    }
    epilogue4<T, EPI>(C, ldc, j * 16 + (l & 15), n0 + (l >> 4) * 4, M, N, total, vec_ok);
  }
}

// ---------------------------------------------------------------------------
// Tiled kernel: 128 x 128 outputs per workgroup, four waves of 64 x 64.
// ---------------------------------------------------------------------------
constexpr int kTile = 128;
constexpr int kRowBytes = 128;            // bytes of K per row per stage (two chunks)
constexpr int kRowStride = kRowBytes + 16;  // padded LDS row

template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                         void* __restrict__ C, int M, int N, int K, long ldx,
                                                         long ldc, int kslice, int aligned, int vec_ok,
                                                         int tiles_m) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int BK = kRowBytes / sizeof(T);  // elements of K per stage
  __shared__ __attribute__((aligned(16))) unsigned char w_lds[kTile * kRowStride];
  __shared__ __attribute__((aligned(16))) unsigned char x_lds[kTile * kRowStride];

  const int tile_m = blockIdx.x % tiles_m;
  const int tile_n = blockIdx.x / tiles_m;
  const int m_base = tile_m * kTile;
  const int n_base = tile_n * kTile;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wn = (wave & 1) * 64;
  const int wm = (wave >> 1) * 64;
  const int row16 = lane & 15;
  const int g = lane >> 4;

  // staging assignment: 8 threads per row (16 bytes each), 32 rows per pass
  const int st_row = threadIdx.x >> 3;
  const int st_col = (threadIdx.x & 7) * A::VEC;

  f32x4 total[4][4];
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      total[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  // Stages of BK elements; kslice is a multiple of BK, so a stage never
  // straddles a slice.  The next stage's global loads are in flight while the
  // current one is multiplied out of LDS.
  vec_t wv[4], xv[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int r = st_row + 32 * p;
    wv[p] = load_vec<T>(W, n_base + r, st_col, K, K, n_base + r < N, aligned);
    xv[p] = load_vec<T>(X, m_base + r, st_col, K, ldx, m_base + r < M, aligned);
  }
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 > 0 && k0 % kslice == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int r = 0; r < 4; ++r) total[i][j][r] = total[i][j][r] + acc[i][j][r];
          acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    __syncthreads();  // previous stage fully consumed
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int r = st_row + 32 * p;
      *reinterpret_cast<vec_t*>(&w_lds[r * kRowStride + st_col * sizeof(T)]) = wv[p];
      *reinterpret_cast<vec_t*>(&x_lds[r * kRowStride + st_col * sizeof(T)]) = xv[p];
    }
    __syncthreads();
    if (k0 + BK < K) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int r = st_row + 32 * p;
        wv[p] = load_vec<T>(W, n_base + r, k0 + BK + st_col, K, K, n_base + r < N, aligned);
        xv[p] = load_vec<T>(X, m_base + r, k0 + BK + st_col, K, ldx, m_base + r < M, aligned);
      }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      // The skinny kernel visits a chunk iff it starts below K; do the same.
      if (k0 + c * A::KCHUNK >= K) break;
      vec_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = *reinterpret_cast<const vec_t*>(&w_lds[(wn + i * 16 + row16) * kRowStride + c * 64 + g * 16]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j] = *reinterpret_cast<const vec_t*>(&x_lds[(wm + j * 16 + row16) * kRowStride + c * 64 + g * 16]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) A::mma(acc[i][j], a[i], b[j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) total[i][j][r] = total[i][j][r] + acc[i][j][r];

#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float t[4] = {total[i][j][0], total[i][j][1], total[i][j][2], total[i][j][3]};
      epilogue4<T, EPI>(C, ldc, m_base + wm + j * 16 + row16, n_base + wn + i * 16 + g * 4, M, N, t, vec_ok);
    }
}

template <typename T, int EPI>
int launch_gemm(const void* X, const void* W, void* C, int M, int N, int K, long ldx, long ldc, hipStream_t stream) {
  const int kslice = kslice_for(K);
  const int nslices = (K + kslice - 1) / kslice;
  constexpr int VEC = Atom<T>::VEC;
  const int aligned = (K % VEC == 0) && (ldx % VEC == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(W) % 16 == 0);
  const size_t out_size = (EPI == kStore) ? sizeof(T) : sizeof(float);
  const int vec_ok = (ldc % 4 == 0) && (reinterpret_cast<uintptr_t>(C) % (4 * out_size) == 0);
  const T* x = reinterpret_cast<const T*>(X);
  const T* w = reinterpret_cast<const T*>(W);
  if (M <= 64) {
    const int mt = (M + 15) / 16;
    const int nw = nslices >= 8 ? 8 : 4;
    dim3 grid((N + 15) / 16);
    const size_t lds = (size_t)nslices * mt * 256 * sizeof(float);
#define LS_SKINNY(MT_, NW_)                                                                            \
  hipLaunchKernelGGL((gemm_skinny_kernel<T, MT_, NW_, EPI>), grid, dim3(NW_ * 64), lds, stream, x, w, C, M, N, K, \
                     ldx, ldc, kslice, aligned, vec_ok)
    if (nw == 8) {
      if (mt == 1) LS_SKINNY(1, 8); else if (mt == 2) LS_SKINNY(2, 8); else if (mt == 3) LS_SKINNY(3, 8); else LS_SKINNY(4, 8);
    } else {
      if (mt == 1) LS_SKINNY(1, 4); else if (mt == 2) LS_SKINNY(2, 4); else if (mt == 3) LS_SKINNY(3, 4); else LS_SKINNY(4, 4);
    }
#undef LS_SKINNY
  } else {
    const int tiles_m = (M + kTile - 1) / kTile;
    const int tiles_n = (N + kTile - 1) / kTile;
    hipLaunchKernelGGL((gemm_tiled_kernel<T, EPI>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, x, w, C, M, N, K,
                       ldx, ldc, kslice, aligned, vec_ok, tiles_m);
  }
  return check_launch("gemm");
}

}  // namespace ls

// dtype: 0 float32, 1 bfloat16.  epilogue: 0 store in dtype, 1 store float,
// 2 add to float.  X [M,K] with ldx elements per row, W [N,K] contiguous,
// C [M,N] with ldc elements per row.
extern "C" int ls_gemm(int dtype, int epilogue, const void* X, const void* W, void* C, int M, int N, int K, long ldx,
                       long ldc, void* stream) {
  using namespace ls;
  LS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: sizes must be positive, got M=%d N=%d K=%d", M, N, K);
  LS_REQUIRE(ldx >= K && ldc >= N, "gemm: row strides ldx=%ld ldc=%ld are shorter than K=%d / N=%d", ldx, ldc, K, N);
  LS_REQUIRE(X && W && C, "gemm: null operand");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define LS_GEMM_CASE(T_)                                                             \
  switch (epilogue) {                                                                \
    case kStore: return launch_gemm<T_, kStore>(X, W, C, M, N, K, ldx, ldc, s);      \
    case kStoreF32: return launch_gemm<T_, kStoreF32>(X, W, C, M, N, K, ldx, ldc, s); \
    case kAddF32: return launch_gemm<T_, kAddF32>(X, W, C, M, N, K, ldx, ldc, s);    \
    default: return fail("gemm: unknown epilogue %d", epilogue);                     \
  }
  if (dtype == kF32) { LS_GEMM_CASE(float) }
  if (dtype == kBF16) { LS_GEMM_CASE(bf16_t) }
#undef LS_GEMM_CASE
  return fail("gemm: unknown dtype %d", dtype);
}

extern "C" int ls_gemm_kslice(int K) { return ls::kslice_for(K); }
