// Shared device helpers for the gfx950 kernels: element types, the MFMA
// "atom" that every contraction is built from, cross-lane reductions with a
// fixed order, and launch checking.
//
// Numerics contract shared by all kernels: a value that belongs to one row
// (one token, one query) is reduced in an order that depends on compile-time
// constants and the row's own sizes only -- never on the number of rows in
// the launch or on where the row sits in a tile.  There are no atomics on
// results and no split of a reduction across workgroups other than the
// fixed, position-anchored splits that a separate kernel folds in ascending
// order.  Floating-point contraction is switched off for the whole library
// (-ffp-contract=off): a fused multiply-add appears only where fmaf is
// written, so the same expression gives the same bits in every kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ls {

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kWave = 64;
constexpr float kNegSentinel = -1e30f;  // finite "minus infinity" of the softmax

enum DType : int { kF32 = 0, kBF16 = 1 };

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return static_cast<float>(x); }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
// float -> bfloat16 is round-to-nearest-even (LLVM fptrunc semantics).
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return static_cast<bf16_t>(x); }

// ---------------------------------------------------------------------------
// The contraction atom.  One "chunk" is 64 bytes of K per row: a lane holds
// 16 bytes of it (VEC elements) at element offset VEC * (lane / 16), for row
// (lane % 16) of its operand.  mma() adds the 16x16 product of two such
// operands to a 16x16 float accumulator of which a lane holds four entries:
// column (lane % 16) of the second operand, rows 4 * (lane / 16) + {0,1,2,3}
// of the first.
//   bf16:  one v_mfma_f32_16x16x32_bf16 (32 K per chunk).
//   f32:   four v_mfma_f32_16x16x4_f32 (16 K per chunk) -- full 32-bit
//          products and sums, no reduced-precision matrix mode.
// ---------------------------------------------------------------------------
template <typename T> struct Atom;

template <> struct Atom<bf16_t> {
  static constexpr int VEC = 8;
  static constexpr int KCHUNK = 32;
  typedef bf16x8 vec_t;
  static __device__ __forceinline__ vec_t zero() { return vec_t{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ void mma(f32x4& acc, const vec_t& a, const vec_t& b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
};

template <> struct Atom<float> {
  static constexpr int VEC = 4;
  static constexpr int KCHUNK = 16;
  typedef f32x4 vec_t;
  static __device__ __forceinline__ vec_t zero() { return vec_t{0.f, 0.f, 0.f, 0.f}; }
  static __device__ __forceinline__ void mma(f32x4& acc, const vec_t& a, const vec_t& b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], acc, 0, 0, 0);
  }
};

// Load VEC elements of row `row` at element offset `k` of a row-major matrix
// with `ld` elements per row, zero where the row is not `ok` or k >= limit.
// `aligned` (uniform) says every row start and k are 16-byte aligned and
// limit is a multiple of VEC; the load is then unconditional (from a clamped
// address) and the zero is selected afterwards, so a run of such loads can
// be in flight together.
template <typename T>
__device__ __forceinline__ typename Atom<T>::vec_t load_vec(const T* __restrict__ base, long row, int k,
                                                            int limit, long ld, bool ok, bool aligned) {
  typedef typename Atom<T>::vec_t vec_t;
  constexpr int VEC = Atom<T>::VEC;
  const bool valid = ok && k < limit;
  if (aligned) {
    const T* p = base + (valid ? row * ld + k : 0);
    vec_t v = *reinterpret_cast<const vec_t*>(p);
    return valid ? v : Atom<T>::zero();
  }
  vec_t v = Atom<T>::zero();
  if (valid) {
    const T* p = base + row * ld + k;
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      if (k + e < limit) v[e] = p[e];
  }
  return v;
}

// Sum / max over the four lanes {l, l^16, l^32, l^48}; every lane of the
// four ends with the same bits because each step adds a pair commutatively.
__device__ __forceinline__ float quad16_sum(float v) {
  v = v + __shfl_xor(v, 16, kWave);
  v = v + __shfl_xor(v, 32, kWave);
  return v;
}
__device__ __forceinline__ float quad16_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  v = fmaxf(v, __shfl_xor(v, 32, kWave));
  return v;
}

// Butterfly sum over all 64 lanes, same bits in every lane.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 1; m < kWave; m <<= 1) v = v + __shfl_xor(v, m, kWave);
  return v;
}

// Sum of squares of a float row as every kernel that normalises computes it:
// thread t of 256 adds the squares of the elements 1024*c + 4*t + {0,1,2,3},
// c = 0, 1, ... in ascending order; then a butterfly over the wave (wave_sum)
// and the four wave sums in wave order.  This returns the thread's part.
__device__ __forceinline__ float row_sumsq_part(const float* __restrict__ src, int width, int t, bool vec_ok) {
  float part = 0.f;
  for (int base = 4 * t; base < width; base += 1024) {
    if (vec_ok && base + 3 < width) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(src + base);
#pragma unroll
      for (int e = 0; e < 4; ++e) part = part + v[e] * v[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (base + e < width) {
          const float v = src[base + e];
          part = part + v * v;
        }
    }
  }
  return part;
}

// One head of one token: optional RMSNorm over the head (weight != nullptr),
// then the half-split rotation of its first `rot` elements.  One wave runs it
// in two phases, so that a caller can put other loads between them:
// head_load brings the lane's elements (e = lane, lane + 64, ...), their norm
// weights and rotation factors into registers; head_finish does the
// arithmetic and hands the results to `dst(e, value)`.  `y` is an LDS row of
// d floats private to the wave.  The sum of squares: lane l adds x[l]^2,
// x[l+64]^2, ... ascending, then a butterfly over the wave.  Every kernel
// that normalises a head goes through these two, so a head has the same bits
// wherever it is processed.
constexpr int kMaxHeadDim = 256;
constexpr int kHeadPerLane = kMaxHeadDim / 64;
struct HeadVec {
  float x[kHeadPerLane], w[kHeadPerLane], c[kHeadPerLane], s[kHeadPerLane];
};

template <typename T>
__device__ __forceinline__ void head_load(HeadVec& h, const T* src, int d, const float* __restrict__ weight,
                                          const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                          int pos, int rot, int lane) {
  const int half = rot / 2;
#pragma unroll
  for (int i = 0; i < kHeadPerLane; ++i) {
    const int e = lane + 64 * i;
    const bool in = e < d;
    h.x[i] = in ? to_f32(src[e]) : 0.f;
    h.w[i] = (weight && in) ? weight[e] : 1.f;
    h.c[i] = 1.f;
    h.s[i] = 0.f;
    if (cos_table && e < rot) {
      const int idx = e < half ? e : e - half;
      h.c[i] = cos_table[(long)pos * half + idx];
      h.s[i] = sin_table[(long)pos * half + idx];
    }
  }
}

template <typename T, typename Dst>
__device__ __forceinline__ void head_finish(const HeadVec& h, int d, bool normed, float eps, bool rotated, int rot,
                                            float* __restrict__ y, int lane, Dst dst) {
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < kHeadPerLane; ++i) {
    const int e = lane + 64 * i;
    if (e < d) {
      y[e] = h.x[i];
      part = part + h.x[i] * h.x[i];
    }
  }
  if (normed) {
    const float total = wave_sum(part);
    const float scale = 1.0f / sqrtf(total / (float)d + eps);
#pragma unroll
    for (int i = 0; i < kHeadPerLane; ++i) {
      const int e = lane + 64 * i;
      if (e < d) y[e] = (h.x[i] * scale) * h.w[i];
    }
  }
  // The staging row is private to this wave: order its writes before the
  // reads of other lanes without a workgroup barrier.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int half = rot / 2;
#pragma unroll
  for (int i = 0; i < kHeadPerLane; ++i) {
    const int e = lane + 64 * i;
    if (e >= d) continue;
    float v = y[e];
    if (rotated && e < rot) {
      const int idx = e < half ? e : e - half;
      const float lo = y[idx];
      const float hi = y[idx + half];
      v = e < half ? lo * h.c[i] - hi * h.s[i] : hi * h.c[i] + lo * h.s[i];
    }
    dst(e, from_f32<T>(v));
  }
  // the row may be reused by the caller for its next head
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

}  // namespace ls

// Error reporting across the C interface: every entry point returns 0 or a
// negative code and leaves a message that ls_last_error() of the same library
// returns.  Each shared library defines ls_last_error() once through
// LS_DEFINE_ERROR_API.
#include <stdarg.h>
#include <stdio.h>
namespace ls {
inline char g_error[1024] = {0};
inline int fail(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
  return -1;
}
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: %s", what, hipGetErrorString(e));
  return 0;
}
}  // namespace ls

#define LS_DEFINE_ERROR_API \
  extern "C" const char* ls_last_error() { return ls::g_error; }

#define LS_REQUIRE(cond, ...)                   \
  do {                                          \
    if (!(cond)) return ls::fail(__VA_ARGS__);  \
  } while (0)
