// Temperature / nucleus sampling on the device.
//
// The procedure is the host sampler's (reference engine/sampler/philox.py:71-98), in float64:
//   v = double(float(logit) / T);  w = exp(v - max v);  S = sum w
//   tokens ordered by (weight descending, id ascending); c(e) = sum of the weights up to e in that order
//   nucleus: the shortest head whose c reaches p * S is kept (all of it when p >= 1); H = its c
//   the draw u * H picks the first token whose c reaches it.
// The host sorts; here the token is found without a sort.  Weights are a monotone function of the float
// v, so the order is that of v's bit pattern, and "the first token whose c reaches t" is found by
// walking down that pattern four bits at a time: one pass over the row sums the weights of the sixteen
// candidates for the next four bits, the sums are taken from the top until the target is reached, and
// after eight passes the float value is known; tokens that share it have the same weight and are counted
// off in the order of their ids.  Every sum has a fixed order (a thread's elements in ascending order, a
// butterfly over the wave, the waves in order), so a row gives the same token every time.  The sums are
// not the host's (it adds in sorted order), so a draw that lands within rounding of a token's boundary
// can fall to the neighbour; nothing else differs.  Distinct float values whose weights round to the
// same double (values below 1e-16 of each other, next to zero) are ordered by value here, by id there.
//
// One workgroup of 1,024 threads a row; the weights and the order keys of a row are kept in a scratch
// buffer the caller brings (12 bytes a token and row).  In a pass a thread adds each of its tokens' weights
// to the thread's own slot of the token's candidate in LDS (sixteen slots a thread, no two threads share
// one, so no atomics and a fixed order); the slots of a candidate are then summed over the block.

#include <hip/hip_runtime.h>

#include "common.h"
#include "core_api.h"

namespace ls {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;
constexpr int kBatch = 8;  // loads a thread has in flight in the passes over a row

__device__ __forceinline__ unsigned int order_key(float f) {  // ascending in f; -0 counts as +0
  const unsigned int b = __float_as_uint(f + 0.0f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// The same total in every thread: butterfly over the wave, then the waves' sums in wave order.
__device__ __forceinline__ double block_sum(double v, double* __restrict__ wave_sums) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off);
  __syncthreads();  // wave_sums may still be read from the call before
  if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = v;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) total = total + wave_sums[w];
  return total;
}

struct Found {
  int token;       // the first token, in the order of the sort, whose cumulative weight reaches the target
  double reached;  // that cumulative weight
};

// `slots`: 16 * kSampleThreads doubles (candidate b of thread t at slots[b * kSampleThreads + t]: a wave's lanes
// fall on different banks whatever their candidates are); `shared_d`: 16 * kSampleWaves doubles; `shared_i`:
// kSampleThreads + 8 ints.
__device__ Found first_reaching(const unsigned int* __restrict__ keys, const double* __restrict__ weights, int vocab,
                                double target, double* __restrict__ slots, double* __restrict__ shared_d,
                                int* __restrict__ shared_i) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  unsigned int prefix = 0;   // the bits of the key that are known, in their place
  double above = 0.0;        // weights of the keys that are larger than every key with this prefix
  for (int shift = 28; shift >= 0; shift -= 4) {
#pragma unroll
    for (int b = 0; b < 16; ++b) slots[b * kSampleThreads + threadIdx.x] = 0.0;
    const unsigned int known = shift == 28 ? 0u : (0xffffffffu << (shift + 4));
    // eight tokens' loads at a time, unconditional, so that they are in flight together; the additions
    // keep the order of the ids
    for (int i0 = threadIdx.x; i0 < vocab; i0 += kBatch * kSampleThreads) {
      unsigned int key[kBatch];
      double w[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = min(i0 + u * kSampleThreads, vocab - 1);
        key[u] = keys[i];
        w[u] = weights[i];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (i0 + u * kSampleThreads >= vocab || (key[u] & known) != prefix) continue;
        double* slot = &slots[((key[u] >> shift) & 15) * kSampleThreads + threadIdx.x];
        *slot = *slot + w[u];
      }
    }
    double sums[16];
#pragma unroll
    for (int b = 0; b < 16; ++b) {
      sums[b] = slots[b * kSampleThreads + threadIdx.x];
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) sums[b] = sums[b] + __shfl_xor(sums[b], off);
    }
    __syncthreads();  // shared_d may still be read from the level before
    if (lane == 0) {
#pragma unroll
      for (int b = 0; b < 16; ++b) shared_d[wave * 16 + b] = sums[b];
    }
    __syncthreads();
    // every thread walks the sixteen sums from the top (the same arithmetic in all of them)
    int chosen = -1, lowest = 0;
    double passed = above;
    for (int b = 15; b >= 0; --b) {
      double s = 0.0;
#pragma unroll
      for (int w = 0; w < kSampleWaves; ++w) s = s + shared_d[w * 16 + b];
      if (!(s > 0.0)) continue;
      lowest = b;
      if (passed + s >= target) {
        chosen = b;
        break;
      }
      passed = passed + s;
    }
    if (chosen < 0) {
      // rounding left the target just above the last sum: the end of the range is meant.  `passed` counts
      // the lowest candidate in; take it out again by walking once more (the same in every thread).
      chosen = lowest;
      passed = above;
      for (int b = 15; b > lowest; --b) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kSampleWaves; ++w) s = s + shared_d[w * 16 + b];
        if (s > 0.0) passed = passed + s;
      }
    }
    above = passed;
    prefix |= (unsigned int)chosen << shift;
  }
  // Tokens whose key is `prefix` share one weight; count them off in the order of their ids.  A thread
  // takes a run of neighbouring ids.
  const int per = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int begin = min(vocab, (int)threadIdx.x * per), end = min(vocab, begin + per);
  int mine = 0, last_tie = -1;
  for (int i0 = begin; i0 < end; i0 += kBatch) {
    unsigned int key[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) key[u] = keys[min(i0 + u, vocab - 1)];
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (i0 + u < end && key[u] == prefix) {
        ++mine;
        last_tie = i0 + u;
      }
  }
  double tie_weight = last_tie >= 0 ? weights[last_tie] : 0.0;
  __syncthreads();
  shared_i[threadIdx.x] = mine;
  // any tie's weight (they are equal): the largest over the block, zero where a thread has none
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) tie_weight = fmax(tie_weight, __shfl_xor(tie_weight, off));
  if (lane == 0) shared_d[wave] = tie_weight;
  __syncthreads();
  double w_tie = 0.0;
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) w_tie = fmax(w_tie, shared_d[w]);
  int before = 0, ties = 0;
  for (int t = 0; t < kSampleThreads; ++t) {
    const int c = shared_i[t];
    if (t < (int)threadIdx.x) before += c;
    ties += c;
  }
  // the m-th tie is the first whose cumulative weight above + m * w reaches the target
  int m = 1;
  if (w_tie > 0.0 && target > above + w_tie) {
    const double need = ceil((target - above) / w_tie);
    m = need >= (double)ties ? ties : (int)need;
    if (m < 1) m = 1;
  }
  if (m > ties) m = ties;
  __syncthreads();
  if (mine > 0 && before < m && m <= before + mine) {
    int seen = before;
    for (int i = begin; i < end; ++i)
      if (keys[i] == prefix && ++seen == m) {
        shared_i[kSampleThreads] = i;
        break;
      }
  }
  if (ties == 0 && threadIdx.x == 0) shared_i[kSampleThreads] = 0;  // an empty row cannot happen; stay in range
  __syncthreads();
  Found found;
  found.token = shared_i[kSampleThreads];
  found.reached = above + (double)m * w_tie;
  __syncthreads();
  return found;
}

// One row's request: which row of the logits, its temperature and nucleus, and the key and counter of
// its draw (32 bytes, as the host packs them).
struct SampleRow {
  int row;
  float temperature;
  double top_p;
  unsigned int key0, key1;   // the two halves of seed XOR k(uid)
  unsigned int pos_lo, pos_hi;
};

// Philox-4x32 with ten rounds; the draw is the first output word times 2^-32 (reference
// engine/sampler/philox.py:9-61; sampling/philox.py is the same in Python).
__device__ __forceinline__ double philox_uniform(unsigned int k0, unsigned int k1, unsigned int c0, unsigned int c1) {
  unsigned int c2 = 0u, c3 = 0u;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const unsigned long long p0 = 0xD2511F53ull * c0;
    const unsigned long long p1 = 0xCD9E8D57ull * c2;
    const unsigned int n0 = (unsigned int)(p1 >> 32) ^ c1 ^ k0;
    const unsigned int n1 = (unsigned int)p1;
    const unsigned int n2 = (unsigned int)(p0 >> 32) ^ c3 ^ k1;
    const unsigned int n3 = (unsigned int)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    if (round + 1 < 10) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
  }
  return (double)c0 * 2.3283064365386963e-10;  // 2^-32, exact
}

__global__ __launch_bounds__(kSampleThreads) void sample_top_p_kernel(
    const float* __restrict__ logits, long ld, const SampleRow* __restrict__ requests, int* __restrict__ out,
    double* __restrict__ scratch_weights, unsigned int* __restrict__ scratch_keys, int vocab) {
  extern __shared__ __attribute__((aligned(16))) double slots[];  // [16][kSampleThreads]
  __shared__ double shared_d[16 * kSampleWaves];
  __shared__ int shared_i[kSampleThreads + 8];
  __shared__ float wave_max[kSampleWaves];
  const int r = blockIdx.x;
  const SampleRow request = requests[r];
  const float* row = logits + (long)request.row * ld;
  const float t = request.temperature;
  double* weights = scratch_weights + (long)r * vocab;
  unsigned int* keys = scratch_keys + (long)r * vocab;

  float top = -INFINITY;
  for (int i0 = threadIdx.x; i0 < vocab; i0 += kBatch * kSampleThreads) {
    float x[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) x[u] = row[min(i0 + u * kSampleThreads, vocab - 1)];  // (a repeated token changes no maximum)
#pragma unroll
    for (int u = 0; u < kBatch; ++u) top = fmaxf(top, x[u] / t);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) top = fmaxf(top, __shfl_xor(top, off));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = top;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) top = fmaxf(top, wave_max[w]);
  const double v_max = (double)top;

  double part = 0.0;
  for (int i0 = threadIdx.x; i0 < vocab; i0 += kBatch * kSampleThreads) {
    float x[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) x[u] = row[min(i0 + u * kSampleThreads, vocab - 1)];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kSampleThreads;
      if (i >= vocab) continue;
      const float f = x[u] / t;
      const double w = exp((double)f - v_max);
      weights[i] = w;
      keys[i] = order_key(f);
      part = part + w;
    }
  }
  const double total = block_sum(part, shared_d);  // (its barriers also publish weights and keys to the block)

  double head = total;
  const double p = request.top_p;
  if (p < 1.0) head = first_reaching(keys, weights, vocab, p * total, slots, shared_d, shared_i).reached;
  // the draw in the word of the counter that the third counter word 0 names (index 0 of the host's uniform())
  const double u = philox_uniform(request.key0, request.key1, request.pos_lo, request.pos_hi);
  const Found pick = first_reaching(keys, weights, vocab, u * head, slots, shared_d, shared_i);
  if (threadIdx.x == 0) out[r] = pick.token;
}

}  // namespace ls

// Sample one token for each of `n` rows.  `requests`: n records of 32 bytes on the device (int row of `logits`,
// float temperature > 0, double top_p, then four unsigned words: the two halves of seed XOR k(uid) and the two
// halves of the position); token ids to out[i].  `logits`: float [.][ld], `vocab` columns.  `scratch`: n * vocab * 12
// bytes, 8-byte aligned (the rows' weights as doubles, then their order keys).
extern "C" int ls_sample_top_p(const float* logits, long ld, const void* requests, int* out, void* scratch, int n,
                               int vocab, void* stream) {
  using namespace ls;
  static_assert(sizeof(SampleRow) == 32, "the host packs 32 bytes a row");
  LS_REQUIRE(n > 0 && vocab > 0 && ld >= vocab, "sample: bad sizes (n=%d vocab=%d ld=%ld)", n, vocab, ld);
  LS_REQUIRE(logits && requests && out && scratch, "sample: null operand");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(scratch) % 8 == 0 && reinterpret_cast<uintptr_t>(requests) % 8 == 0,
             "sample: the scratch buffer and the requests must be 8-byte aligned");
  constexpr size_t lds = (size_t)16 * kSampleThreads * sizeof(double);  // 128 KB: granted per kernel, once
  static int granted = 0;                                              // 0 unknown, 1 yes, -1 no
  if (granted == 0) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_top_p_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) (void)hipGetLastError();
    granted = e == hipSuccess ? 1 : -1;
  }
  if (granted != 1) return fail("sample: the device does not grant %zu bytes of LDS to a workgroup", lds);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  double* weights = reinterpret_cast<double*>(scratch);
  unsigned int* keys = reinterpret_cast<unsigned int*>(weights + (size_t)n * vocab);
  hipLaunchKernelGGL(sample_top_p_kernel, dim3(n), dim3(kSampleThreads), lds, s, logits, ld,
                     reinterpret_cast<const SampleRow*>(requests), out, weights, keys, vocab);
  return check_launch("sample");
}
