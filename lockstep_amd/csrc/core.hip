// Row-wise kernels of the step: embedding gather, RMSNorm of the residual
// stream, per-head norm + rotation + cache write, SwiGLU, arg-max.
//
// The residual stream is float in both precisions; everything that goes into
// a matrix product is in the compute dtype T (float or bfloat16).  All
// reductions are per row with an order fixed by the row's width alone.

#include <mutex>

#include "common.h"
#include "core_api.h"

#ifdef LS_MUTANTS
__device__ int ls_mutants_dev = 0;  // external linkage: the compiler must not assume it stays zero
#endif

namespace ls {

// ---------------------------------------------------------------------------
// Embedding: h[t, :] = float(E[token[t], :]).  A token id outside the table
// writes zeros (the host rejects such ids before the launch; the kernel must
// not fault on them).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                                    float* __restrict__ out, int vocab, int width, long ld_out) {
  const int t = blockIdx.x;
  const int id = tokens[t];
  const bool ok = id >= 0 && id < vocab;
  const T* row = table + (long)(ok ? id : 0) * width;
  float* dst = out + (long)t * ld_out;
  for (int e = threadIdx.x; e < width; e += blockDim.x) dst[e] = ok ? to_f32(row[e]) : 0.f;
}

// ---------------------------------------------------------------------------
// RMSNorm over rows of the float residual stream:
//   y = (x * 1/sqrt(sum(x^2)/N + eps)) * w      (all in float), stored as T.
// One workgroup per output row.  Thread i sums x[i]^2, x[i+256]^2, ... in
// ascending order; a wave adds its lanes by butterfly; the four wave sums are
// added in wave order.  `rows` (optional) picks the input row of each output.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                      T* __restrict__ out, const int* __restrict__ rows, int width,
                                                      long ldx, long ld_out, float eps) {
  __shared__ float wave_part[4];
  const int r_out = blockIdx.x;
  const long r_in = rows ? rows[r_out] : r_out;
  const float* src = x + r_in * ldx;
  T* dst = out + (long)r_out * ld_out;
  const bool vec_ok = (ldx & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  // Rows of up to 4,096 elements stay in registers between the two passes, and their weights are
  // requested before the reduction, so the kernel waits for memory once.  The sum is row_sumsq_part's.
  constexpr int KEEP = 4;
  const bool fast = vec_ok && width <= KEEP * 1024 && (width & 3) == 0 &&
                    (reinterpret_cast<uintptr_t>(weight) & 15) == 0 && (ld_out & 3) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & (4 * sizeof(T) - 1)) == 0;
  if (fast) {
    f32x4 v[KEEP], w[KEEP];
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < KEEP; ++c) {
      const int base = 1024 * c + 4 * (int)threadIdx.x;
      const bool in = base < width;
      v[c] = in ? *reinterpret_cast<const f32x4*>(src + base) : f32x4{0.f, 0.f, 0.f, 0.f};
      w[c] = in ? *reinterpret_cast<const f32x4*>(weight + base) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int c = 0; c < KEEP; ++c)
      if (1024 * c + 4 * (int)threadIdx.x < width) {
#pragma unroll
        for (int e = 0; e < 4; ++e) part = part + v[c][e] * v[c][e];
      }
    part = wave_sum(part);
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
    __syncthreads();
    float total = ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
    if (LS_MUTANT_DEVICE(kMutantNormByRows) && gridDim.x > 4)
      total = ((wave_part[3] + wave_part[2]) + wave_part[1]) + wave_part[0];
    const float scale = 1.0f / sqrtf(total / (float)width + eps);
#pragma unroll
    for (int c = 0; c < KEEP; ++c) {
      const int base = 1024 * c + 4 * (int)threadIdx.x;
      if (base >= width) continue;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (v[c][e] * scale) * w[c][e];
      if (sizeof(T) == 2) {
        bf16x4 b;
        b[0] = (bf16_t)o[0]; b[1] = (bf16_t)o[1]; b[2] = (bf16_t)o[2]; b[3] = (bf16_t)o[3];
        *reinterpret_cast<bf16x4*>(dst + base) = b;
      } else {
        *reinterpret_cast<f32x4*>(dst + base) = f32x4{o[0], o[1], o[2], o[3]};
      }
    }
    return;
  }
  float part = wave_sum(row_sumsq_part(src, width, threadIdx.x, vec_ok));
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  float total = ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
  if (LS_MUTANT_DEVICE(kMutantNormByRows) && gridDim.x > 4)
    total = ((wave_part[3] + wave_part[2]) + wave_part[1]) + wave_part[0];
  const float scale = 1.0f / sqrtf(total / (float)width + eps);
  for (int e = threadIdx.x; e < width; e += 256) dst[e] = from_f32<T>((src[e] * scale) * weight[e]);
}

// ---------------------------------------------------------------------------
// Per (token, head) of the fused q|k|v projection output:
//   q, k heads: optional RMSNorm over the head (one [d] weight for all
//   heads), then optional half rotation of the first `rot` dims with the
//   pair (i, i + rot/2):  lo' = lo*c - hi*s,  hi' = hi*c + lo*s  at the
//   token's absolute position; q is written back in place, k goes to the
//   key pages [page][kv head][slot][d];
//   v heads: copied to the transposed value pages [page][kv head][d][slot].
// One wave per (token, head); sums of squares: lane i adds x[i]^2,
// x[i+64]^2, ... ascending, then a butterfly over the wave.
// ---------------------------------------------------------------------------

struct SeqMeta {  // one per sequence of the step (all int32)
  int q_off;      // first packed row
  int q_len;      // rows in this step
  int q_start;    // absolute position of the first row
  int kv_len;     // q_start + q_len
  int table_row;  // row of the block table
  int reserved[3];
};

template <typename T, int PASSES>
__global__ __launch_bounds__(256) void qk_rope_kv_kernel(
    T* __restrict__ qkv, long ld, int nq, int nkv, int d, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const SeqMeta* __restrict__ seqs, const int* __restrict__ table, int table_stride, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int page_size, int write_kv, int n_tokens) {
  const int head_blocks = (int)(((long)n_tokens * (write_kv ? nq + nkv : nq) + 15) / 16);
  if ((int)blockIdx.x >= head_blocks) {
    // Values: a workgroup copies 16 consecutive tokens of the batch.  Sixteen neighbouring lanes
    // hold the same columns of 16 tokens, so where the tokens are neighbours in a page their
    // elements leave as whole runs of 16 slots of the transposed page.  A thread loads one 16-byte run of
    // its token's row (a workgroup takes 16 such runs of its 16 tokens) and stores its elements one by one.
    constexpr int RUN = 16 / (int)sizeof(T);
    const int width = nkv * d;  // the value heads of a token are contiguous; so are the rows of a page
    const int col_blocks = (width + 16 * RUN - 1) / (16 * RUN);
    const int vb = (int)blockIdx.x - head_blocks;
    const int j = threadIdx.x & 15;
    const int t = (vb / col_blocks) * 16 + j;
    if (t >= n_tokens) return;
    const int c0 = (vb % col_blocks) * 16 * RUN + (threadIdx.x >> 4) * RUN;
    if (c0 >= width) return;  // (d is a multiple of RUN: a run lies inside the row or outside)
    const int pos = tok_pos[t];
    const SeqMeta sm = seqs[tok_seq[t]];
    const long page = table[(long)sm.table_row * table_stride + pos / page_size];
    if (page < 0) return;
    const int slot = pos % page_size;
    const T* src = qkv + (long)t * ld + (long)(nq + nkv) * d;
    T* dst = v_pages + page * nkv * d * page_size + slot;
    T v[RUN];
    if (sizeof(T) == 2) {
      const bf16x8 run = *reinterpret_cast<const bf16x8*>(src + c0);
#pragma unroll
      for (int u = 0; u < RUN; ++u) v[u] = run[u];
    } else {
      const f32x4 run = *reinterpret_cast<const f32x4*>(src + c0);
#pragma unroll
      for (int u = 0; u < RUN; ++u) v[u] = run[u];
    }
#pragma unroll
    for (int u = 0; u < RUN; ++u) dst[(long)(c0 + u) * page_size] = v[u];
    return;
  }
  // Query and key heads: sixteen lanes a head (see head16_finish), sixteen heads a workgroup.
  const int heads = write_kv ? nq + nkv : nq;  // the value heads are copied by the workgroups above
  const int gl = threadIdx.x & 15;
  const long gid = (long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (gid >= (long)n_tokens * heads) return;  // the whole group leaves
  const int t = (int)(gid / heads);
  const int head = (int)(gid % heads);
  const bool is_q = head < nq;
  T* src = qkv + (long)t * ld + (long)head * d;
  const int pos = tok_pos[t];
  T* dst = src;
  bool held = true;
  if (!is_q) {
    const SeqMeta sm = seqs[tok_seq[t]];
    const long page = table[(long)sm.table_row * table_stride + pos / page_size];
    held = page >= 0;  // the host never schedules a write to a page it does not hold
    dst = k_pages + ((max(page, 0L) * nkv + (head - nq)) * page_size + pos % page_size) * d;
  }
  const float* weight = is_q ? q_weight : k_weight;
  float x[8 * PASSES];
  HeadFactors<PASSES> f;
  head16_load_values<T, PASSES>(x, src, d, gl);
  head16_load_factors<PASSES>(f, d, weight, cos_table, sin_table, pos, rot, gl);
  head16_finish<T, PASSES>(x, f, d, weight != nullptr, eps, cos_table != nullptr, rot, gl, [&](int e0, const T (&v)[8]) LS_INLINED {
    if (held) store8<T>(dst + e0, v);
  });
}

// ---------------------------------------------------------------------------
// SwiGLU: act = (g * 1/(1 + exp(-g))) * u in float; gu [rows, 2*I] holds the
// gates in columns [0, I) and the ups in [I, 2I).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int rows,
                                                     int inter, long ld_in, long ld_out) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * inter) return;
  const long r = idx / inter;
  const int c = (int)(idx % inter);
  const float g = to_f32(gu[r * ld_in + c]);
  const float u = to_f32(gu[r * ld_in + inter + c]);
  const float sig = 1.0f / (1.0f + expf(-g));
  out[r * ld_out + c] = from_f32<T>((g * sig) * u);
}

// ---------------------------------------------------------------------------
// Bias and activation on float rows (the output of a product stored in float):
//   out[m][n] = act(x[m][n] + bias[n])                              plain
//   out[m][n] = act(x[m][n] + bias[n]) * (x[m][N + n] + bias[N + n])  gated (x has 2N columns)
// for parts with biases or with another activation than the product's own SwiGLU epilogue: a
// pass of its own over the rows, slower than an epilogue, but it keeps every such part out of the
// product kernels.  `out` may be `x` itself (plain, float output).  All arithmetic in float.
// ---------------------------------------------------------------------------
enum Activation { kActNone = 0, kActSilu = 1, kActGeluTanh = 2, kActGelu = 3, kActRelu = 4 };

__device__ __forceinline__ float activate(float v, int act) {
  switch (act) {
    case kActSilu: return v * (1.0f / (1.0f + expf(-v)));
    case kActGeluTanh: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    case kActGelu: return 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
    case kActRelu: return fmaxf(v, 0.0f);
    default: return v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bias_act_kernel(const float* __restrict__ x, long ldx,
                                                       const float* __restrict__ bias, T* __restrict__ out, long ldo,
                                                       int rows, int width, int act, int gated) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * width) return;
  const long r = idx / width;
  const int c = (int)(idx % width);
  float v = x[r * ldx + c];
  if (bias) v = v + bias[c];
  v = activate(v, act);
  if (gated) {
    float u = x[r * ldx + width + c];
    if (bias) u = u + bias[width + c];
    v = v * u;
  }
  out[r * ldo + c] = from_f32<T>(v);
}

// ---------------------------------------------------------------------------
// Residual add of a product left as slice sums, then RMSNorm of the new row:
//   h[row] += (P[0][row] + P[1][row] + ...)   (slices ascending, from +0)
//   out[r] = rmsnorm(h[row]) * weight         (skipped when out == nullptr)
// `row` = rows[r] when a row list is given (then only the listed rows are
// touched).  The sums and the norm are those of the separate kernels
// (skinny product's fold and epilogue, rmsnorm_kernel), bit for bit.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ P,
                                                          int slices, int p_rows, const float* __restrict__ weight,
                                                          T* __restrict__ out, const int* __restrict__ rows, int width,
                                                          long ldh, long ld_out, float eps) {
  __shared__ float wave_part[4];
  const int r_out = blockIdx.x;
  const long row = rows ? rows[r_out] : r_out;
  float* hrow = h + row * ldh;
  // requirements checked on the host: width % 4 == 0, 16-byte aligned rows; any width
  f32x4 w_first = f32x4{0.f, 0.f, 0.f, 0.f};  // the weights of the thread's first run, requested before the sums
  if (out != nullptr && 4 * (int)threadIdx.x < width) w_first = *reinterpret_cast<const f32x4*>(weight + 4 * threadIdx.x);
  float part = 0.f;
  constexpr int BATCH = 16;  // slice sums requested together
  for (int base = 4 * threadIdx.x; base < width; base += 1024) {
    f32x4 total = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 old = *reinterpret_cast<const f32x4*>(hrow + base);
    for (int s0 = 0; s0 < slices; s0 += BATCH) {
      f32x4 p[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u)  // clamped: all loads are issued before the first is needed
        p[u] = *reinterpret_cast<const f32x4*>(P + ((long)min(s0 + u, slices - 1) * p_rows + row) * width + base);
#pragma unroll
      for (int u = 0; u < BATCH; ++u)
        if (s0 + u < slices) {
#pragma unroll
          for (int e = 0; e < 4; ++e) total[e] = total[e] + p[u][e];
        }
    }
    f32x4 fresh;
#pragma unroll
    for (int e = 0; e < 4; ++e) fresh[e] = old[e] + total[e];
    *reinterpret_cast<f32x4*>(hrow + base) = fresh;
#pragma unroll
    for (int e = 0; e < 4; ++e) part = part + fresh[e] * fresh[e];
  }
  if (out == nullptr) return;
  part = wave_sum(part);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  const float total = ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
  const float scale = 1.0f / sqrtf(total / (float)width + eps);
  T* dst = out + (long)r_out * ld_out;
  for (int base = 4 * threadIdx.x; base < width; base += 1024) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(hrow + base);  // this thread wrote it above
    const f32x4 w = base == 4 * (int)threadIdx.x ? w_first : *reinterpret_cast<const f32x4*>(weight + base);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[base + e] = from_f32<T>((v[e] * scale) * w[e]);
  }
}

// The same for rows of more than 1,024 elements: 1,024 threads, so that the
// slice sums of a whole row of up to 4,096 elements are requested at once
// (a row is one workgroup's work, and with few rows the kernel's time is that
// of one row).  Thread (c0, t) = (tid / 256, tid % 256) forms the new values
// of the runs 1024 c + 4 t, c = c0, c0 + 4, ...; the squares are then added by
// the threads t of the first four waves over c = 0, 1, ... from LDS, which is
// row_sumsq_part's order.
template <typename T>
__global__ __launch_bounds__(1024) void add_rmsnorm_wide_kernel(float* __restrict__ h, const float* __restrict__ P,
                                                                int slices, int p_rows,
                                                                const float* __restrict__ weight, T* __restrict__ out,
                                                                const int* __restrict__ rows, int width, long ldh,
                                                                long ld_out, float eps) {
  extern __shared__ __attribute__((aligned(16))) float fresh_lds[];  // the new row
  __shared__ float wave_part[4];
  const int r_out = blockIdx.x;
  const long row = rows ? rows[r_out] : r_out;
  float* hrow = h + row * ldh;
  const int t = threadIdx.x & 255;
  const int c0 = threadIdx.x >> 8;
  constexpr int BATCH = 16;  // slice sums requested together
  for (int base = 1024 * c0 + 4 * t; base < width; base += 4096) {
    f32x4 total = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 old = *reinterpret_cast<const f32x4*>(hrow + base);
    for (int s0 = 0; s0 < slices; s0 += BATCH) {
      f32x4 p[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u)  // clamped: all loads are issued before the first is needed
        p[u] = *reinterpret_cast<const f32x4*>(P + ((long)min(s0 + u, slices - 1) * p_rows + row) * width + base);
#pragma unroll
      for (int u = 0; u < BATCH; ++u)
        if (s0 + u < slices) {
#pragma unroll
          for (int e = 0; e < 4; ++e) total[e] = total[e] + p[u][e];
        }
    }
    f32x4 fresh;
#pragma unroll
    for (int e = 0; e < 4; ++e) fresh[e] = old[e] + total[e];
    *reinterpret_cast<f32x4*>(hrow + base) = fresh;
    *reinterpret_cast<f32x4*>(fresh_lds + base) = fresh;
  }
  if (out == nullptr) return;
  __syncthreads();
  if (c0 == 0) {
    float part = 0.f;
    for (int base = 4 * t; base < width; base += 1024) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(fresh_lds + base);
#pragma unroll
      for (int e = 0; e < 4; ++e) part = part + v[e] * v[e];
    }
    part = wave_sum(part);
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  }
  __syncthreads();
  const float total = ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
  const float scale = 1.0f / sqrtf(total / (float)width + eps);
  T* dst = out + (long)r_out * ld_out;
  for (int base = 1024 * c0 + 4 * t; base < width; base += 4096) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(fresh_lds + base);
    const f32x4 w = *reinterpret_cast<const f32x4*>(weight + base);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[base + e] = from_f32<T>((v[e] * scale) * w[e]);
  }
}

// ---------------------------------------------------------------------------
// Arg-max of float rows with the lowest index among equal maxima (NaN never
// wins; a row without a winner gives 0).  A row is cut into chunks of
// kArgmaxChunk elements, one workgroup each, whose winners a second small
// launch reduces; a row of one chunk is finished by the first launch.
// ---------------------------------------------------------------------------
constexpr int kArgmaxChunk = 4096;

__device__ __forceinline__ void argmax_take(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

// Reduce (bv, bi) over the 256 threads of the workgroup; valid in thread 0.
__device__ __forceinline__ void argmax_reduce(float& bv, int& bi) {
  __shared__ float wave_v[4];
  __shared__ int wave_i[4];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_take(bv, bi, ov, oi);
  }
  if ((threadIdx.x & 63) == 0) {
    wave_v[threadIdx.x >> 6] = bv;
    wave_i[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < 4; ++w) argmax_take(bv, bi, wave_v[w], wave_i[w]);
}

__global__ __launch_bounds__(256) void argmax_chunk_kernel(const float* __restrict__ x, int* __restrict__ out,
                                                           float* __restrict__ part_v, int* __restrict__ part_i,
                                                           int width, long ld, int chunks) {
  const float* row = x + (long)blockIdx.y * ld;
  const int lo = blockIdx.x * kArgmaxChunk;
  const int hi = min(width, lo + kArgmaxChunk);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  if ((ld & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // four loads in flight per thread
    constexpr int PER = kArgmaxChunk / (256 * 4);
    f32x4 v[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lo + (j * 256 + threadIdx.x) * 4;
      v[j] = e + 3 < hi ? *reinterpret_cast<const f32x4*>(row + e) : f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (e + 3 >= hi)
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (e + k < hi) v[j][k] = row[e + k];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int e = lo + (j * 256 + threadIdx.x) * 4 + k;
        argmax_take(bv, bi, v[j][k], e < hi ? e : 0x7fffffff);  // padding never wins
      }
  } else {
    for (int e = lo + threadIdx.x; e < hi; e += 256) argmax_take(bv, bi, row[e], e);
  }
  argmax_reduce(bv, bi);
  if (threadIdx.x == 0) {
    if (chunks == 1) {
      out[blockIdx.y] = bi == 0x7fffffff ? 0 : bi;
    } else {
      part_v[(long)blockIdx.y * chunks + blockIdx.x] = bv;
      part_i[(long)blockIdx.y * chunks + blockIdx.x] = bi;
    }
  }
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ part_v,
                                                           const int* __restrict__ part_i, int* __restrict__ out,
                                                           int chunks) {
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 256)
    argmax_take(bv, bi, part_v[(long)blockIdx.x * chunks + c], part_i[(long)blockIdx.x * chunks + c]);
  argmax_reduce(bv, bi);
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// ---------------------------------------------------------------------------
// Between two decode steps that run without the host: every request takes the
// token that was picked for it as its next input, at the next position.  The
// step's metadata (see the engine's upload) is advanced in place: the token
// ids are replaced, and every value named by the table of runs (first, stride,
// count) inside the metadata moves on by one -- token positions, the requests'
// first position and length, and whatever copies of them the parts keep in
// blocks of their own (the host checks that no value is named twice).  The
// picked tokens are also appended to a ring the host reads later:
// ring[step][request], step = *counter, which is incremented.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void advance_decode_kernel(int* __restrict__ meta, int n_seqs, int off_tokens,
                                                             const int* __restrict__ picked, int* __restrict__ ring,
                                                             int* __restrict__ counter, int off_runs, int n_runs) {
  // one workgroup, so that the counter can be read by all of it before one thread moves it on
  const int tid = threadIdx.x;
  const int stride = blockDim.x;
  const int step = *counter;
  for (int i = tid; i < n_seqs; i += stride) {
    const int token = picked[i];
    meta[off_tokens + i] = token;
    ring[(long)step * n_seqs + i] = token;
  }
  for (int r = 0; r < n_runs; ++r) {
    const int first = meta[off_runs + 3 * r], step_ints = meta[off_runs + 3 * r + 1], count = meta[off_runs + 3 * r + 2];
    for (int i = tid; i < count; i += stride) meta[first + step_ints * i] += 1;
  }
  __syncthreads();
  if (tid == 0) *counter = step + 1;
}

}  // namespace ls

LS_DEFINE_ERROR_API

// The entry points that a list of launches may name (the kernels of a layer).
#define LS_CORE_LISTED(X)                                                                                        \
  X(ls_gemm) X(ls_gemm_slices) X(ls_gemm_slices_folded) X(ls_add_rmsnorm) X(ls_rmsnorm) X(ls_qk_rope_kv) X(ls_swiglu) \
  X(ls_bias_act) X(ls_embed)
LS_DEFINE_LISTED_CALLS(LS_CORE_LISTED)

extern "C" int ls_run_list(const long long* words, long n_words, long* failed_at) {
  typedef int (*callee_t)(int, const long long*, int);
  long at = 0;
  while (at < n_words) {
    if (at + 3 > n_words || words[at + 2] < 0 || at + 3 + words[at + 2] > n_words) {
      if (failed_at) *failed_at = at;
      return ls::fail("run_list: the record at word %ld runs past the end of the list", at);
    }
    const callee_t callee = reinterpret_cast<callee_t>(static_cast<uintptr_t>(words[at]));
    const int n = (int)words[at + 2];
    const int code = callee((int)words[at + 1], words + at + 3, n);
    if (code != 0) {
      if (failed_at) *failed_at = at;
      return code;
    }
    at += 3 + n;
  }
  return 0;
}
LS_DEFINE_MUTANT_API

using namespace ls;

extern "C" int ls_embed(int dtype, const int* tokens, const void* table, float* out, int n_tokens, int vocab,
                        int width, long ld_out, void* stream) {
  LS_REQUIRE(n_tokens > 0 && vocab > 0 && width > 0 && ld_out >= width, "embed: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == kF32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n_tokens), dim3(256), 0, s, tokens, (const float*)table, out, vocab,
                       width, ld_out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, s, tokens, (const bf16_t*)table, out,
                       vocab, width, ld_out);
  else
    return fail("embed: unknown dtype %d", dtype);
  return check_launch("embed");
}

extern "C" int ls_rmsnorm(int dtype, const float* x, const float* weight, void* out, const int* rows, int n_rows,
                          int width, long ldx, long ld_out, float eps, void* stream) {
  LS_REQUIRE(n_rows > 0 && width > 0 && ldx >= width && ld_out >= width, "rmsnorm: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == kF32)
    hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(n_rows), dim3(256), 0, s, x, weight, (float*)out, rows, width, ldx,
                       ld_out, eps);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, s, x, weight, (bf16_t*)out, rows, width,
                       ldx, ld_out, eps);
  else
    return fail("rmsnorm: unknown dtype %d", dtype);
  return check_launch("rmsnorm");
}

// h [*, ldh] float: rows (all n_rows first rows, or the listed ones) get the slice sums P [slices][p_rows][width]
// added (ascending), then out [n_rows, ld_out] = rmsnorm of the new rows; out == nullptr: add only.
extern "C" int ls_add_rmsnorm(int dtype, float* h, const float* P, int slices, int p_rows, const float* weight,
                              void* out, const int* rows, int n_rows, int width, long ldh, long ld_out, float eps,
                              void* stream) {
  LS_REQUIRE(n_rows > 0 && width > 0 && slices > 0 && p_rows > 0 && ldh >= width, "add_rmsnorm: bad sizes");
  LS_REQUIRE(width % 4 == 0 && ldh % 4 == 0 && reinterpret_cast<uintptr_t>(h) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(P) % 16 == 0,
             "add_rmsnorm: rows must be 16-byte aligned and a multiple of 4 wide (width %d, ldh %ld)", width, ldh);
  LS_REQUIRE(out == nullptr || (weight != nullptr && ld_out >= width && reinterpret_cast<uintptr_t>(weight) % 16 == 0),
             "add_rmsnorm: the norm needs an aligned weight and an output row of %d elements", width);
  LS_REQUIRE(rows != nullptr || n_rows <= p_rows, "add_rmsnorm: %d rows, the slice sums hold %d", n_rows, p_rows);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype != kF32 && dtype != kBF16) return fail("add_rmsnorm: unknown dtype %d", dtype);
  // wide rows (few of them: the time of the kernel is the time of one row): four times the threads
  const size_t row_bytes = (size_t)width * sizeof(float);
  if (width > 1024 && row_bytes <= 64 * 1024) {
    if (dtype == kF32)
      hipLaunchKernelGGL(add_rmsnorm_wide_kernel<float>, dim3(n_rows), dim3(1024), row_bytes, s, h, P, slices, p_rows,
                         weight, (float*)out, rows, width, ldh, ld_out, eps);
    else
      hipLaunchKernelGGL(add_rmsnorm_wide_kernel<bf16_t>, dim3(n_rows), dim3(1024), row_bytes, s, h, P, slices,
                         p_rows, weight, (bf16_t*)out, rows, width, ldh, ld_out, eps);
    return check_launch("add_rmsnorm");
  }
  if (dtype == kF32)
    hipLaunchKernelGGL(add_rmsnorm_kernel<float>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_rows, weight,
                       (float*)out, rows, width, ldh, ld_out, eps);
  else
    hipLaunchKernelGGL(add_rmsnorm_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_rows, weight,
                       (bf16_t*)out, rows, width, ldh, ld_out, eps);
  return check_launch("add_rmsnorm");
}

extern "C" int ls_qk_rope_kv(int dtype, void* qkv, long ld, int n_tokens, int nq, int nkv, int d,
                             const float* q_weight, const float* k_weight, float eps, const float* cos_table,
                             const float* sin_table, int rot, int table_positions, const int* tok_seq,
                             const int* tok_pos, const void* seqs, const int* table, int table_stride, void* k_pages,
                             void* v_pages, int page_size, int write_kv, void* stream) {
  LS_REQUIRE(n_tokens > 0 && nq >= 0 && nkv >= 0 && d > 0, "qk_rope_kv: bad sizes");
  LS_REQUIRE(d <= kMaxHeadDim, "qk_rope_kv: head_dim %d exceeds the supported maximum %d", d, kMaxHeadDim);
  LS_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "qk_rope_kv: rotary_dim %d must be even and at most head_dim %d",
             rot, d);
  LS_REQUIRE(!cos_table || (sin_table && table_positions > 0), "qk_rope_kv: rotation tables incomplete");
  const int heads = write_kv ? nq + 2 * nkv : nq;
  LS_REQUIRE(ld >= (long)heads * d, "qk_rope_kv: row stride %ld shorter than %d heads of %d", ld, heads, d);
  LS_REQUIRE(!write_kv || (k_pages && v_pages && table && page_size > 0), "qk_rope_kv: cache operands missing");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  LS_REQUIRE(head16_supported(d, rot), "qk_rope_kv: head_dim %d must be a multiple of 8 up to %d and rotary_dim %d even and "
             "at most head_dim", d, kMaxHeadDim, rot);
  const size_t elem = dtype == kF32 ? 4 : 2;
  LS_REQUIRE(reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && (ld * elem) % 16 == 0 && (d * elem) % 16 == 0 &&
                 (!write_kv || reinterpret_cast<uintptr_t>(k_pages) % 16 == 0),
             "qk_rope_kv: rows, heads and pages must be 16-byte aligned (ld=%ld, head_dim=%d)", ld, d);
  LS_REQUIRE((!q_weight || reinterpret_cast<uintptr_t>(q_weight) % 16 == 0) &&
                 (!k_weight || reinterpret_cast<uintptr_t>(k_weight) % 16 == 0) &&
                 (!cos_table || (reinterpret_cast<uintptr_t>(cos_table) % 16 == 0 &&
                                 reinterpret_cast<uintptr_t>(sin_table) % 16 == 0)),
             "qk_rope_kv: norm weights and rotation tables must be 16-byte aligned");
  const long head_blocks = ((long)n_tokens * (write_kv ? nq + nkv : nq) + 15) / 16;
  const long run = 16 / (long)elem;  // elements of a 16-byte run: a workgroup of the value copy takes 16 runs of 16 tokens
  const long value_blocks = write_kv ? (long)((n_tokens + 15) / 16) * (((long)nkv * d + 16 * run - 1) / (16 * run)) : 0;
  dim3 grid((unsigned)(head_blocks + value_blocks));
#define LS_ROPE(T_, P_)                                                                                            \
  hipLaunchKernelGGL((qk_rope_kv_kernel<T_, P_>), grid, dim3(256), 0, s, (T_*)qkv, ld, nq, nkv, d, q_weight, k_weight, \
                     eps, cos_table, sin_table, rot, tok_seq, tok_pos, (const SeqMeta*)seqs, table, table_stride,   \
                     (T_*)k_pages, (T_*)v_pages, page_size, write_kv, n_tokens)
  if (dtype == kF32) {
    if (d > 128) LS_ROPE(float, 2); else LS_ROPE(float, 1);
  } else if (dtype == kBF16) {
    if (d > 128) LS_ROPE(bf16_t, 2); else LS_ROPE(bf16_t, 1);
  } else {
    return fail("qk_rope_kv: unknown dtype %d", dtype);
  }
#undef LS_ROPE
  return check_launch("qk_rope_kv");
}

extern "C" int ls_swiglu(int dtype, const void* gu, void* out, int rows, int inter, long ld_in, long ld_out,
                         void* stream) {
  LS_REQUIRE(rows > 0 && inter > 0 && ld_in >= 2L * inter && ld_out >= inter, "swiglu: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long total = (long)rows * inter;
  dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == kF32)
    hipLaunchKernelGGL(swiglu_kernel<float>, grid, dim3(256), 0, s, (const float*)gu, (float*)out, rows, inter, ld_in,
                       ld_out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)gu, (bf16_t*)out, rows, inter,
                       ld_in, ld_out);
  else
    return fail("swiglu: unknown dtype %d", dtype);
  return check_launch("swiglu");
}

// out_dtype: 0 float32, 1 bfloat16.  act: 0 none, 1 SiLU, 2 GELU (tanh form), 3 GELU (erf form), 4 ReLU.
// x float [rows][ldx] with `width` columns (2 * width when gated), bias float [width] ([2 * width] when
// gated) or null, out [rows][ldo] of out_dtype; out may be x (not gated, float32).
extern "C" int ls_bias_act(int out_dtype, const float* x, long ldx, const float* bias, void* out, long ldo, int rows,
                           int width, int act, int gated, void* stream) {
  using namespace ls;
  LS_REQUIRE(rows > 0 && width > 0 && ldo >= width && ldx >= (gated ? 2 * width : width), "bias_act: bad sizes");
  LS_REQUIRE(act >= 0 && act <= 4, "bias_act: unknown activation %d", act);
  LS_REQUIRE(!(gated && (const void*)x == out), "bias_act: a gated pass cannot work in place");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long total = (long)rows * width;
  dim3 grid((unsigned)((total + 255) / 256));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(bias_act_kernel<float>, grid, dim3(256), 0, s, x, ldx, bias, (float*)out, ldo, rows, width, act,
                       gated);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(bias_act_kernel<bf16_t>, grid, dim3(256), 0, s, x, ldx, bias, (bf16_t*)out, ldo, rows, width,
                       act, gated);
  else
    return fail("bias_act: unknown dtype %d", out_dtype);
  return check_launch("bias_act");
}

// Chunks a row of this width is cut into; scratch must hold 2 * rows * chunks 4-byte words when chunks > 1.
extern "C" int ls_argmax_chunks(int width) { return (width + kArgmaxChunk - 1) / kArgmaxChunk; }

extern "C" int ls_argmax(const float* x, int* out, int rows, int width, long ld, void* scratch, long scratch_words,
                         void* stream) {
  LS_REQUIRE(rows > 0 && width > 0 && ld >= width, "argmax: bad sizes");
  const int chunks = ls_argmax_chunks(width);
  LS_REQUIRE(chunks == 1 || (scratch != nullptr && scratch_words >= 2L * rows * chunks),
             "argmax: scratch of %ld words is too small for %d rows of %d chunks", scratch_words, rows, chunks);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* part_v = reinterpret_cast<float*>(scratch);
  int* part_i = reinterpret_cast<int*>(scratch) + (long)rows * chunks;
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(chunks, rows), dim3(256), 0, s, x, out, part_v, part_i, width, ld,
                     chunks);
  if (chunks > 1) hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(256), 0, s, part_v, part_i, out, chunks);
  return check_launch("argmax");
}

// ---------------------------------------------------------------------------
// Arg-max for callers that cannot allocate (see core_api.h).  The chunks'
// winners go to `argmax_scratch`, an array in the library's device image:
// values in the first LS_ARGMAX_STATIC_PAIRS words, indices in the second.
// In host code the array's name is only a stand-in for the symbol; the
// address of each GPU's own copy is asked from the runtime once per device
// (g_argmax_scratch_ptr) and only that pointer is handed to kernels.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned int argmax_scratch[2 * LS_ARGMAX_STATIC_PAIRS];

namespace ls {
constexpr int kMaxDevices = 64;
static void* g_argmax_scratch_ptr[kMaxDevices] = {nullptr};
static std::mutex g_argmax_scratch_mutex;

// The current device's copy of argmax_scratch; looked up at the first call on that device.
static int argmax_scratch_of_current_device(void** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail("argmax_static: hipGetDevice: %s", hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices) return fail("argmax_static: device %d is outside [0, %d)", device, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_argmax_scratch_mutex);
  if (g_argmax_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(argmax_scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail("argmax_static: hipGetSymbolAddress on device %d: %s", device, hipGetErrorString(e));
    g_argmax_scratch_ptr[device] = ptr;
  }
  *out = g_argmax_scratch_ptr[device];
  return 0;
}
}  // namespace ls

extern "C" int ls_argmax_static(const float* x, int* out, int rows, int width, long ld, void* stream) {
  LS_REQUIRE(x && out && rows > 0 && width > 0 && ld >= width, "argmax_static: bad operands or sizes");
  const int chunks = ls_argmax_chunks(width);
  LS_REQUIRE((long)rows * chunks <= (long)LS_ARGMAX_STATIC_PAIRS,
             "argmax_static: %d rows of %d chunks need %ld scratch entries, the static array holds %d "
             "(use ls_argmax with a scratch buffer of your own)",
             rows, chunks, (long)rows * chunks, LS_ARGMAX_STATIC_PAIRS);
  void* ptr = nullptr;
  if (int code = argmax_scratch_of_current_device(&ptr)) return code;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // both halves sized for the capacity, so the layout does not depend on the call
  float* part_v = reinterpret_cast<float*>(ptr);
  int* part_i = reinterpret_cast<int*>(ptr) + LS_ARGMAX_STATIC_PAIRS;
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(chunks, rows), dim3(256), 0, s, x, out, part_v, part_i, width, ld,
                     chunks);
  if (chunks > 1) hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(256), 0, s, part_v, part_i, out, chunks);
  return check_launch("argmax_static");
}

// meta [meta_ints]: the step's uploaded metadata; picked [n_seqs]: the tokens chosen for the requests; ring
// [steps][n_seqs] and counter: where the loop's output goes.  The table of n_runs runs (first, stride, count)
// lies at meta[off_runs]; the caller has checked that every run stays inside meta and outside the table.
extern "C" int ls_advance_decode(int* meta, long meta_ints, int n_seqs, int off_tokens, const int* picked, int* ring,
                                 int* counter, int off_runs, int n_runs, void* stream) {
  LS_REQUIRE(meta && picked && ring && counter && n_seqs > 0, "advance_decode: bad operands");
  LS_REQUIRE(off_tokens >= 0 && off_tokens + (long)n_seqs <= meta_ints, "advance_decode: the token ids lie outside the metadata");
  LS_REQUIRE(n_runs >= 0 && off_runs >= 0 && off_runs + 3L * n_runs <= meta_ints,
             "advance_decode: the table of %d runs at %d lies outside the %ld ints of metadata", n_runs, off_runs, meta_ints);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(advance_decode_kernel, dim3(1), dim3(256), 0, s, meta, n_seqs, off_tokens, picked, ring, counter,
                     off_runs, n_runs);
  return check_launch("advance_decode");
}
