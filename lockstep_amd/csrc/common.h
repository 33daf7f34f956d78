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

}  // namespace ls
// Every lambda of a kernel is part of the kernel's body: one that the compiler leaves as a function of its own
// is called through the stack, with everything it captures kept in scratch memory (seen in the float instances
// of the fused decode kernel: 75 us a launch instead of 13).
#define LS_INLINED __attribute__((always_inline))

namespace ls {

// The exponential of the softmax and of the fold over attention splits: the library routine on the
// 32-bit path, the hardware's on the bfloat16 path.  One definition for every kernel that folds.
template <typename T> __device__ __forceinline__ float softmax_exp(float x);
template <> __device__ __forceinline__ float softmax_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float softmax_exp<bf16_t>(float x) { return __expf(x); }

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

// One head of one token: optional RMSNorm over the head, then the half-split
// rotation of its first `rot` elements.  Sixteen neighbouring lanes (a group)
// process a head; lane i of the group holds the elements [8i, 8i + 8) and, for
// heads of more than 128 elements (PASSES == 2), also [128 + 8i, 128 + 8i + 8),
// so that values, weights and rotation factors move as 16-byte vectors and no
// LDS is needed.  The sum of squares: a lane adds its squares in ascending
// order of the element, then the group adds over the lanes i+8, i+4, i+2,
// i+1 (mod 16), which leaves the same bits in all of its lanes.  The partner
// of the rotation, half = rot/2 elements away, is fetched from its lane by a
// shuffle (one per element where half is a multiple of 8, a slower gather
// otherwise).  Every
// kernel that normalises a head goes through these functions, so a head has
// the same bits wherever it is processed.
constexpr int kMaxHeadDim = 256;

__host__ __device__ inline bool head16_supported(int d, int rot) {
  return d % 8 == 0 && d <= kMaxHeadDim && rot % 2 == 0 && rot <= d;
}

template <int PASSES>
struct HeadFactors {  // what does not depend on the head's values
  float w[8 * PASSES], c[8 * PASSES], s[8 * PASSES];
};

template <int N>
__device__ __forceinline__ void load_floats8(float* dst, const float* __restrict__ src, bool ok, float fill) {
  if (ok) {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(src);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dst[j] = lo[j];
      dst[4 + j] = hi[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[j] = fill;
  }
}

// gl: the lane's index in its group of 16.  weight / tables may be nullptr.
template <int PASSES>
__device__ __forceinline__ void head16_load_factors(HeadFactors<PASSES>& f, int d, const float* __restrict__ weight,
                                                    const float* __restrict__ cos_table,
                                                    const float* __restrict__ sin_table, int pos, int rot, int gl) {
  const int half = rot / 2;
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int e0 = 128 * p + 8 * gl;
    load_floats8<8>(f.w + 8 * p, weight + (weight ? e0 : 0), weight != nullptr && e0 < d, 1.f);
    if ((half & 7) == 0) {  // uniform: a run of eight lies on one side of the half
      const bool turn = cos_table != nullptr && e0 < rot;
      const int idx = e0 < half ? e0 : e0 - half;
      const long at = turn ? (long)pos * half + idx : 0;
      load_floats8<8>(f.c + 8 * p, cos_table + at, turn, 1.f);
      load_floats8<8>(f.s + 8 * p, sin_table + at, turn, 0.f);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int e = e0 + j;
        const bool turn = cos_table != nullptr && e < rot;
        const long at = turn ? (long)pos * half + (e < half ? e : e - half) : 0;
        f.c[8 * p + j] = turn ? cos_table[at] : 1.f;
        f.s[8 * p + j] = turn ? sin_table[at] : 0.f;
      }
    }
  }
}

// src: the head's first element; 16-byte aligned.
template <typename T, int PASSES>
__device__ __forceinline__ void head16_load_values(float (&x)[8 * PASSES], const T* src, int d, int gl) {
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int e0 = 128 * p + 8 * gl;
    if (e0 < d) {
      if (sizeof(T) == 2) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(src + e0);
#pragma unroll
        for (int j = 0; j < 8; ++j) x[8 * p + j] = to_f32(v[j]);
      } else {
        load_floats8<8>(x + 8 * p, reinterpret_cast<const float*>(src) + e0, true, 0.f);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[8 * p + j] = 0.f;
    }
  }
}

// The value `v` of the lane K places on in the caller's row of sixteen lanes, the row taken as a ring (a
// data-parallel move inside the row: no trip through LDS as a fetch from an arbitrary lane takes).
template <int K>
__device__ __forceinline__ float row16_rotated(float v) {
  static_assert(K >= 1 && K <= 15, "a rotation inside a row of sixteen");
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + K, 0xf, 0xf, false));
}

// Value of `v` in lane `from` (0..15) of the caller's group.
__device__ __forceinline__ float group16_get(float v, int from) {
  return __shfl(v, (threadIdx.x & 48) | from, kWave);
}

// dst(e0, vals): called for each run of eight finished elements [e0, e0 + 8) of the head.
template <typename T, int PASSES, typename Dst>
__device__ __forceinline__ void head16_finish(const float (&x)[8 * PASSES], const HeadFactors<PASSES>& f, int d,
                                              bool normed, float eps, bool rotated, int rot, int gl, Dst dst) {
  float y[8 * PASSES];
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < 8 * PASSES; ++i) part = part + x[i] * x[i];  // elements past d are zeros
  if (normed) {
    // part_i + part_(i+8), then + the sum four lanes on, two, one: after each step the sums repeat with the
    // step's period, so the lane k on and the lane k back hold the same value and a rotation of the row of
    // sixteen lanes in either direction gives the same bits as a fetch from lane (gl + k) & 15
    part = part + row16_rotated<8>(part);
    part = part + row16_rotated<4>(part);
    part = part + row16_rotated<2>(part);
    part = part + row16_rotated<1>(part);
    const float scale = 1.0f / sqrtf(part / (float)d + eps);
#pragma unroll
    for (int i = 0; i < 8 * PASSES; ++i) y[i] = (x[i] * scale) * f.w[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8 * PASSES; ++i) y[i] = x[i];
  }
  const int half = rot / 2;
  const bool run_aligned = (half & 7) == 0;  // uniform
  if (PASSES == 1 && rotated && run_aligned) {  // uniform: a lane's eight partners are the eight of one other lane
    const int e0 = 8 * gl;
    const bool lower = e0 < half, turns = e0 < rot;
    const int lanes_apart = half >> 3;
    const int from = (((threadIdx.x & 63 & ~15) | ((gl + (lower ? lanes_apart : 16 - lanes_apart)) & 15))) << 2;
    float other[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) other[j] = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(y[j])));
    T out[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // lower half: y c - other s; upper half: y c + other s (a - b and a + (-b) are the same bits)
      const float s = lower ? -f.s[j] : f.s[j];
      const float turned = y[j] * f.c[j] + other[j] * s;
      out[j] = from_f32<T>(turns ? turned : y[j]);
    }
    if (e0 < d) dst(e0, out);
    return;
  }
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int e0 = 128 * p + 8 * gl;
    T out[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int e = e0 + j;
      float v = y[8 * p + j];
      if (rotated) {  // uniform
        // the partner lies half elements above (for the lower half) or below
        const bool lower = e < half;
        const int partner = lower ? e + half : e - half;
        const int from_lane = (partner & 127) >> 3;
        const int from_pass = e < rot ? partner >> 7 : 0;
        float other = 0.f;
        if (run_aligned) {  // the partner has the same place j in its lane's run
          other = group16_get(y[j], from_lane);
          if (PASSES == 2) {
            const float other1 = group16_get(y[8 + j], from_lane);
            other = from_pass ? other1 : other;
          }
        } else {
#pragma unroll
          for (int k = 0; k < 8 * PASSES; ++k) {
            const float cand = group16_get(y[k], from_lane);
            other = (k == 8 * from_pass + (partner & 7)) ? cand : other;
          }
        }
        if (e < rot) {
          const float lo = lower ? v : other;
          const float hi = lower ? other : v;
          v = lower ? lo * f.c[8 * p + j] - hi * f.s[8 * p + j] : hi * f.c[8 * p + j] + lo * f.s[8 * p + j];
        }
      }
      out[j] = from_f32<T>(v);
    }
    if (e0 < d) dst(e0, out);
  }
}

// Store eight elements at a 16-byte aligned address.
template <typename T>
__device__ __forceinline__ void store8(T* at, const T (&v)[8]) {
  if (sizeof(T) == 2) {
    bf16x8 w;
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = v[j];
    *reinterpret_cast<bf16x8*>(at) = w;
  } else {
    float* p = reinterpret_cast<float*>(at);
    *reinterpret_cast<f32x4*>(p) = f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
  }
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

// Entry points called from a list of 8-byte words, one word an argument (an integer, a pointer, or a float's
// bits in the low half): a caller that repeats many launches hands the whole list over in one call instead of
// crossing into the library once a launch.  A library names its listed entry points once,
//   #define MY_LISTED(X) X(ls_gemm) X(ls_rmsnorm) ...
//   LS_DEFINE_LISTED_CALLS(MY_LISTED)
// which defines ls_listed_index(name) (-1: not listed) and ls_call_listed(index, words, n).
#include <string.h>

#include <type_traits>
#include <utility>
namespace ls {
template <typename T>
inline T word_as(long long w) {
  if constexpr (std::is_pointer_v<T>) {
    return reinterpret_cast<T>(static_cast<uintptr_t>(w));
  } else if constexpr (std::is_same_v<T, float>) {
    const unsigned int bits = static_cast<unsigned int>(w);
    float f;
    memcpy(&f, &bits, sizeof(f));
    return f;
  } else {
    static_assert(std::is_integral_v<T>, "listed entry points take integers, pointers and floats");
    return static_cast<T>(w);
  }
}
template <typename... A, size_t... I>
inline int call_words(int (*fn)(A...), const long long* w, std::index_sequence<I...>) {
  return fn(word_as<A>(w[I])...);
}
template <typename... A>
inline int call_words(const char* name, int (*fn)(A...), const long long* w, int n) {
  if (n != (int)sizeof...(A)) return fail("%s takes %d arguments, the list brings %d", name, (int)sizeof...(A), n);
  return call_words(fn, w, std::index_sequence_for<A...>{});
}
#define LS_LISTED_NAME(f) \
  if (strcmp(name, #f) == 0) return at; \
  ++at;
#define LS_LISTED_CALL(f) \
  if (index == at++) return ls::call_words(#f, &f, words, n);
#define LS_DEFINE_LISTED_CALLS(ENTRIES)                                             \
  extern "C" int ls_listed_index(const char* name) {                                \
    int at = 0;                                                                     \
    ENTRIES(LS_LISTED_NAME)                                                         \
    return -1;                                                                      \
  }                                                                                 \
  extern "C" int ls_call_listed(int index, const long long* words, int n) {         \
    int at = 0;                                                                     \
    ENTRIES(LS_LISTED_CALL)                                                         \
    return ls::fail("there is no listed entry point %d", index);                    \
  }

// Compute units of the current device (asked once per device).
inline int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
}  // namespace ls

#define LS_DEFINE_ERROR_API \
  extern "C" const char* ls_last_error() { return ls::g_error; }

// Positive controls.  A library built with -DLS_MUTANTS (the tests build one beside the product
// library, under a name of its own) carries deliberately wrong variants of a few reductions, each
// switched on by a bit of a mask that ls_set_mutants() sets: variants whose summation order
// depends on how many rows or work items a launch has.  They exist so that the tests of batch
// independence can be shown to fail when the property is broken.  Without the define the
// conditions below are constant false and nothing of this is in the product library.
namespace ls {
// bits of the mask, core library
constexpr int kMutantKsliceByRows = 1;  // the skinny product cuts K into other slices above 16 rows
constexpr int kMutantNormByRows = 2;    // RMSNorm adds its wave sums in another order in launches of more than four rows
constexpr int kMutantSampleChunksByRows = 4;  // the sampler cuts a row into fewer chunks when the call has many rows
constexpr int kMutantReversedFoldInProduct = 8;  // the product that folds attention splits itself folds them from the last to the first
// bits of the mask, attention libraries
constexpr int kMutantReversedFold = 1;  // the combine kernel folds the splits from the last to the first
}  // namespace ls
#ifdef LS_MUTANTS
namespace ls {
inline int g_mutants = 0;  // host-side copy of the mask
}
#define LS_MUTANT_HOST(bit) ((ls::g_mutants & (bit)) != 0)
#define LS_MUTANT_DEVICE(bit) ((ls_mutants_dev & (bit)) != 0)
#define LS_DEFINE_MUTANT_API                                                                       \
  extern "C" int ls_set_mutants(int mask) {                                                        \
    ls::g_mutants = mask;                                                                          \
    hipError_t e = hipMemcpyToSymbol(HIP_SYMBOL(ls_mutants_dev), &mask, sizeof(int));              \
    if (e != hipSuccess) return ls::fail("set_mutants: %s", hipGetErrorString(e));                 \
    return 0;                                                                                      \
  }
#else
#define LS_MUTANT_HOST(bit) false
#define LS_MUTANT_DEVICE(bit) false
#define LS_DEFINE_MUTANT_API
#endif

#define LS_REQUIRE(cond, ...)                   \
  do {                                          \
    if (!(cond)) return ls::fail(__VA_ARGS__);  \
  } while (0)
