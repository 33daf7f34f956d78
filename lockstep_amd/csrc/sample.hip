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
// A row is always cut into kChunks runs of neighbouring tokens, whatever else the call samples: which
// elements a thread adds and how the chunks' sums are folded are functions of the vocabulary alone, so a
// row gives the same token beside any number of other rows.  A workgroup takes one chunk, or (many rows)
// several chunks of a row one after the other, each exactly as a workgroup of its own would.  Every step
// of the walk is a launch of its own: a launch reads the sums the launch before left for every chunk, adds
// them up in chunk order (every workgroup of the row does the same arithmetic, so they agree without
// talking to each other), and leaves its own chunks' sums.  The weights and the order keys of a row are
// kept in a scratch buffer the caller brings.  In a pass a thread adds each of its tokens' weights to the
// thread's own slot of the token's candidate in LDS (sixteen slots a thread, no two threads share one, so
// no atomics and a fixed order); the slots of a candidate are then summed over the workgroup.

#include <hip/hip_runtime.h>

#include "common.h"
#include "core_api.h"

#include <algorithm>

#ifndef LS_SAMPLE_WORKGROUPS_A_CU
#define LS_SAMPLE_WORKGROUPS_A_CU 4  // workgroups a CU that a launch aims at: with more rows a workgroup walks several chunks
#endif

namespace ls {

constexpr int kSampleThreads = 256;
constexpr int kSampleWaves = kSampleThreads / 64;
constexpr int kChunks = 32;  // chunks a row is cut into, always
constexpr int kBatch = 8;    // loads a thread has in flight in the passes over its chunk

__device__ __forceinline__ unsigned int order_key(float f) {  // ascending in f; -0 counts as +0
  const unsigned int b = __float_as_uint(f + 0.0f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// One row's request: which row of the logits, its temperature and nucleus, and the key and counter of
// its draw (32 bytes, as the host packs them).
struct SampleRow {
  int row;
  float temperature;
  unsigned int top_p_lo, top_p_hi;  // the double, in two words: records may lie at any multiple of four bytes
  unsigned int key0, key1;          // the two halves of seed XOR k(uid)
  unsigned int pos_lo, pos_hi;      // (pos_lo moves on by one a token where steps run without the host)
  __device__ __forceinline__ double top_p() const { return __hiloint2double((int)top_p_hi, (int)top_p_lo); }
};

// Where a walk stands: the bits of the key that are known (in their place), the weights of all keys above
// every key with these bits, and what the walk looks for.
struct SearchState {
  double target, above;
  unsigned int prefix;
  int pad;
};

struct Found {
  double reached;  // the cumulative weight of the token that was found
  int token;
  int pad;
};

// What the launches of one call leave for each other, per row (and per chunk where it says so).
struct SampleScratch {
  int chunks;             // chunks a row (kChunks; a mutant of the tests' control library makes it follow the rows)
  double* weights;        // [n][vocab]
  unsigned int* keys;     // [n][vocab]
  float* part_max;        // [n][kChunks]
  double* part_sum;       // [n][kChunks]
  double* part_level;     // [2][n][kChunks][16]: the candidates' sums of a chunk, by the parity of the level
  SearchState* state;     // [2 walks][2 parities][n]
  int* tie_count;         // [n][kChunks]
  double* tie_weight;     // [n][kChunks]
  Found* found;           // [2 walks][n]
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

// All kernels below: grid (g, n) with g <= chunks; the workgroup (x, r) takes the chunks x, x + g, ... of row r,
// one after the other, each as if it were alone.

// the largest float(logit) / T of a chunk
__global__ __launch_bounds__(kSampleThreads) void sample_max_kernel(const float* __restrict__ logits, long ld,
                                                                    const SampleRow* __restrict__ requests,
                                                                    SampleScratch sc, int vocab, int chunk_len) {
  __shared__ float wave_max[kSampleWaves];
  const int r = blockIdx.y;
  const SampleRow request = requests[r];
  const float* row = logits + (long)request.row * ld;
  for (int c = blockIdx.x; c < sc.chunks; c += gridDim.x) {
    const int begin = min(vocab, c * chunk_len), end = min(vocab, begin + chunk_len);
    float top = -INFINITY;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kBatch * kSampleThreads) {
      float x[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) x[u] = row[min(i0 + u * kSampleThreads, end - 1)];  // (a repeated token changes no maximum)
#pragma unroll
      for (int u = 0; u < kBatch; ++u) top = fmaxf(top, x[u] / request.temperature);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) top = fmaxf(top, __shfl_xor(top, off));
    __syncthreads();  // wave_max may still be read for the chunk before
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = top;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
      for (int w = 0; w < kSampleWaves; ++w) top = fmaxf(top, wave_max[w]);
      sc.part_max[r * sc.chunks + c] = top;
    }
  }
}

// weights and order keys of a chunk, and the sum of its weights
__global__ __launch_bounds__(kSampleThreads) void sample_exp_kernel(const float* __restrict__ logits, long ld,
                                                                    const SampleRow* __restrict__ requests,
                                                                    SampleScratch sc, int vocab, int chunk_len) {
  __shared__ double wave_sums[kSampleWaves];
  const int r = blockIdx.y;
  const SampleRow request = requests[r];
  const float* row = logits + (long)request.row * ld;
  double* weights = sc.weights + (long)r * vocab;
  unsigned int* keys = sc.keys + (long)r * vocab;
  float top = -INFINITY;
  for (int k = 0; k < sc.chunks; ++k) top = fmaxf(top, sc.part_max[r * sc.chunks + k]);
  const double v_max = (double)top;
  for (int c = blockIdx.x; c < sc.chunks; c += gridDim.x) {
    const int begin = min(vocab, c * chunk_len), end = min(vocab, begin + chunk_len);
    double part = 0.0;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kBatch * kSampleThreads) {
      float x[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) x[u] = row[min(i0 + u * kSampleThreads, end - 1)];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int i = i0 + u * kSampleThreads;
        if (i >= end) continue;
        const float f = x[u] / request.temperature;
        const double w = exp((double)f - v_max);
        weights[i] = w;
        keys[i] = order_key(f);
        part = part + w;
      }
    }
    const double total = block_sum(part, wave_sums);
    if (threadIdx.x == 0) sc.part_sum[r * sc.chunks + c] = total;
  }
}

// The state of walk `walk` of row r after level `level - 1`, from the state after level `level - 2` (which
// the launch before left, or the start of the walk) and the sums of level `level - 1`.  Every thread of
// every workgroup of the row computes it with the same arithmetic.
// `staged`: kChunks * 16 doubles of LDS; all threads of the workgroup call this together.
__device__ SearchState state_before_level(const SampleScratch& sc, const SampleRow& request, int n, int r, int walk,
                                          int level, double* __restrict__ staged) {
  SearchState st;
  if (level == 0) {
    double total = 0.0;
    for (int k = 0; k < sc.chunks; ++k) total = total + sc.part_sum[r * sc.chunks + k];
    if (walk == 0) {
      st.target = request.top_p() * total;  // the nucleus: the shortest head that reaches top_p
    } else {
      const double head = request.top_p() < 1.0 ? sc.found[0 * n + r].reached : total;
      st.target = philox_uniform(request.key0, request.key1, request.pos_lo, request.pos_hi) * head;
    }
    st.above = 0.0;
    st.prefix = 0u;
    st.pad = 0;
    return st;
  }
  st = sc.state[(walk * 2 + (level & 1)) * n + r];  // after level - 2 (parity of level - 2 = parity of level)
  const int shift = 28 - 4 * (level - 1);
  // the chunks' sums of level - 1 into LDS with one round of loads, then every thread walks them
  const double* from = sc.part_level + ((long)((level - 1) & 1) * n + r) * sc.chunks * 16;
  for (int i = threadIdx.x; i < sc.chunks * 16; i += kSampleThreads) staged[i] = from[i];
  __syncthreads();
  const double* sums = staged;
  int chosen = -1, lowest = 0;
  double passed = st.above;
  for (int b = 15; b >= 0; --b) {
    double s = 0.0;
    for (int k = 0; k < sc.chunks; ++k) s = s + sums[k * 16 + b];
    if (!(s > 0.0)) continue;
    lowest = b;
    if (passed + s >= st.target) {
      chosen = b;
      break;
    }
    passed = passed + s;
  }
  if (chosen < 0) {
    // rounding left the target just above the last sum: the end of the range is meant.  `passed` counts
    // the lowest candidate in; take it out again by walking once more.
    chosen = lowest;
    passed = st.above;
    for (int b = 15; b > lowest; --b) {
      double s = 0.0;
      for (int k = 0; k < sc.chunks; ++k) s = s + sums[k * 16 + b];
      if (s > 0.0) passed = passed + s;
    }
  }
  st.above = passed;
  st.prefix |= (unsigned int)chosen << shift;
  return st;
}

// levels 0 to 7: the sums of a chunk's weights for the sixteen candidates of this level's four bits, among the
// tokens whose known bits fit.
__global__ __launch_bounds__(kSampleThreads) void sample_level_kernel(const SampleRow* __restrict__ requests,
                                                                      SampleScratch sc, int n, int vocab, int chunk_len,
                                                                      int walk, int level) {
  __shared__ double slots[16 * kSampleThreads];  // candidate b of thread t at slots[b * kSampleThreads + t]
  __shared__ double wave_sums[kSampleWaves * 16];
  const int r = blockIdx.y;
  const SampleRow request = requests[r];
  if (walk == 0 && !(request.top_p() < 1.0)) return;  // the whole row is the head
  __shared__ double staged[kChunks * 16];
  const SearchState st = state_before_level(sc, request, n, r, walk, level, staged);
  if (blockIdx.x == 0 && threadIdx.x == 0) sc.state[(walk * 2 + ((level + 1) & 1)) * n + r] = st;  // parity of level - 1
  const unsigned int* keys = sc.keys + (long)r * vocab;
  const double* weights = sc.weights + (long)r * vocab;
  const int shift = 28 - 4 * level;
  const unsigned int known = level == 0 ? 0u : (0xffffffffu << (shift + 4));
  for (int c = blockIdx.x; c < sc.chunks; c += gridDim.x) {
#pragma unroll
    for (int b = 0; b < 16; ++b) slots[b * kSampleThreads + threadIdx.x] = 0.0;
    const int begin = min(vocab, c * chunk_len), end = min(vocab, begin + chunk_len);
    // eight tokens' keys at a time, unconditional, so that the loads are in flight together; then the weights
    // of those whose known bits fit (from the second level on these are few, and the others' weights are
    // never fetched); the additions keep the order of the ids
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kBatch * kSampleThreads) {
      unsigned int key[kBatch];
      double w[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) key[u] = keys[min(i0 + u * kSampleThreads, end - 1)];
      bool fits[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) fits[u] = i0 + u * kSampleThreads < end && (key[u] & known) == st.prefix;
#pragma unroll
      for (int u = 0; u < kBatch; ++u) w[u] = fits[u] ? weights[i0 + u * kSampleThreads] : 0.0;
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (!fits[u]) continue;
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
    __syncthreads();  // wave_sums may still be read for the chunk before
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int b = 0; b < 16; ++b) wave_sums[(threadIdx.x >> 6) * 16 + b] = sums[b];
    }
    __syncthreads();
    if (threadIdx.x < 16) {
      double s = 0.0;
#pragma unroll
      for (int w = 0; w < kSampleWaves; ++w) s = s + wave_sums[w * 16 + threadIdx.x];
      sc.part_level[(((long)(level & 1) * n + r) * sc.chunks + c) * 16 + threadIdx.x] = s;
    }
  }
}

// after level 7: the key is known; how many tokens of the chunk have it, and their weight
__global__ __launch_bounds__(kSampleThreads) void sample_tie_count_kernel(const SampleRow* __restrict__ requests,
                                                                          SampleScratch sc, int n, int vocab,
                                                                          int chunk_len, int walk) {
  __shared__ int wave_count[kSampleWaves];
  __shared__ double wave_weight[kSampleWaves];
  const int r = blockIdx.y;
  const SampleRow request = requests[r];
  if (walk == 0 && !(request.top_p() < 1.0)) return;
  __shared__ double staged[kChunks * 16];
  const SearchState st = state_before_level(sc, request, n, r, walk, 8, staged);
  if (blockIdx.x == 0 && threadIdx.x == 0) sc.state[(walk * 2 + 1) * n + r] = st;  // after level 7
  const unsigned int* keys = sc.keys + (long)r * vocab;
  const double* weights = sc.weights + (long)r * vocab;
  for (int c = blockIdx.x; c < sc.chunks; c += gridDim.x) {
    const int begin = min(vocab, c * chunk_len), end = min(vocab, begin + chunk_len);
    int mine = 0, last_tie = -1;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kBatch * kSampleThreads) {
      unsigned int key[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) key[u] = keys[min(i0 + u * kSampleThreads, end - 1)];
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (i0 + u * kSampleThreads < end && key[u] == st.prefix) {
          ++mine;
          last_tie = i0 + u * kSampleThreads;
        }
    }
    double weight = last_tie >= 0 ? weights[last_tie] : 0.0;  // they are equal: any of them
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      mine += __shfl_xor(mine, off);
      weight = fmax(weight, __shfl_xor(weight, off));
    }
    __syncthreads();  // the wave values may still be read for the chunk before
    if ((threadIdx.x & 63) == 0) {
      wave_count[threadIdx.x >> 6] = mine;
      wave_weight[threadIdx.x >> 6] = weight;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int count = 0;
      double w = 0.0;
#pragma unroll
      for (int k = 0; k < kSampleWaves; ++k) {
        count += wave_count[k];
        w = fmax(w, wave_weight[k]);
      }
      sc.tie_count[r * sc.chunks + c] = count;
      sc.tie_weight[r * sc.chunks + c] = w;
    }
  }
}

// tokens that share the key are counted off in the order of their ids; the chunk that holds the one that is
// meant finds it.
__global__ __launch_bounds__(kSampleThreads) void sample_tie_pick_kernel(const SampleRow* __restrict__ requests,
                                                                         SampleScratch sc, int n, int vocab,
                                                                         int chunk_len, int walk, int* __restrict__ out,
                                                                         int scatter) {
  __shared__ int counts[kSampleThreads];
  __shared__ int picked;
  const int r = blockIdx.y;
  const SampleRow request = requests[r];
  if (walk == 0 && !(request.top_p() < 1.0)) return;
  const SearchState st = sc.state[(walk * 2 + 1) * n + r];
  int ties = 0;
  double w_tie = 0.0;
  for (int k = 0; k < sc.chunks; ++k) {
    ties += sc.tie_count[r * sc.chunks + k];
    w_tie = fmax(w_tie, sc.tie_weight[r * sc.chunks + k]);
  }
  // the m-th tie is the first whose cumulative weight above + m * w reaches the target
  int m = 1;
  if (w_tie > 0.0 && st.target > st.above + w_tie) {
    const double need = ceil((st.target - st.above) / w_tie);
    m = need >= (double)ties ? ties : (int)need;
    if (m < 1) m = 1;
  }
  if (m > ties) m = ties;
  const unsigned int* keys = sc.keys + (long)r * vocab;
  for (int c = blockIdx.x; c < sc.chunks; c += gridDim.x) {
    int before = 0;
    for (int k = 0; k < c; ++k) before += sc.tie_count[r * sc.chunks + k];
    const int mine_total = sc.tie_count[r * sc.chunks + c];
    if (!(before < m && m <= before + mine_total)) continue;  // another chunk holds it (uniform for the workgroup)
    // a thread takes a run of neighbouring ids of the chunk
    const int begin = min(vocab, c * chunk_len), end = min(vocab, begin + chunk_len);
    const int per = (chunk_len + kSampleThreads - 1) / kSampleThreads;
    const int lo = min(end, begin + (int)threadIdx.x * per), hi = min(end, lo + per);
    int mine = 0;
    for (int i = lo; i < hi; ++i) mine += keys[i] == st.prefix ? 1 : 0;
    counts[threadIdx.x] = mine;
    __syncthreads();
    int ahead = before;
    for (int t = 0; t < (int)threadIdx.x; ++t) ahead += counts[t];
    if (mine > 0 && ahead < m && m <= ahead + mine) {
      int seen = ahead;
      for (int i = lo; i < hi; ++i)
        if (keys[i] == st.prefix && ++seen == m) {
          picked = i;
          break;
        }
      Found found;
      found.reached = st.above + (double)m * w_tie;
      found.token = picked;
      found.pad = 0;
      sc.found[walk * n + r] = found;
      if (walk == 1) out[scatter ? request.row : r] = picked;
    }
    return;  // one chunk holds it: nothing is left to look for
  }
}

}  // namespace ls

static size_t align_up(size_t bytes) { return (bytes + 255) / 256 * 256; }

// Bytes of scratch that ls_sample_top_p needs for n rows of a vocabulary.
extern "C" long ls_sample_scratch_bytes(int n, int vocab) {
  using namespace ls;
  if (n <= 0 || vocab <= 0) return 0;
  size_t total = align_up((size_t)n * vocab * sizeof(double)) + align_up((size_t)n * vocab * sizeof(unsigned int));
  total += align_up((size_t)n * kChunks * sizeof(float)) + align_up((size_t)n * kChunks * sizeof(double));
  total += align_up((size_t)2 * n * kChunks * 16 * sizeof(double)) + align_up((size_t)4 * n * sizeof(SearchState));
  total += align_up((size_t)n * kChunks * sizeof(int)) + align_up((size_t)n * kChunks * sizeof(double));
  total += align_up((size_t)2 * n * sizeof(Found));
  return (long)total;
}

// Sample one token for each of `n` rows.  `requests`: n records of 32 bytes on the device (int row of `logits`,
// float temperature > 0, double top_p (low word first), then four unsigned words: the two halves of seed XOR k(uid) and the two
// halves of the position); token ids to out[i], or with `scatter` to out[row of the record].  `logits`: float
// [.][ld], `vocab` columns.  `scratch`: ls_sample_scratch_bytes(n, vocab) bytes, 256-byte aligned.  `any_nucleus`:
// 0 if every top_p is >= 1 (the launches that look for the nucleus are then left out).
extern "C" int ls_sample_top_p(const float* logits, long ld, const void* requests, int* out, void* scratch,
                               long scratch_bytes, int n, int vocab, int any_nucleus, int scatter, void* stream) {
  using namespace ls;
  static_assert(sizeof(SampleRow) == 32, "the host packs 32 bytes a row");
  LS_REQUIRE(n > 0 && vocab > 0 && ld >= vocab, "sample: bad sizes (n=%d vocab=%d ld=%ld)", n, vocab, ld);
  LS_REQUIRE(logits && requests && out && scratch, "sample: null operand");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(scratch) % 256 == 0 && reinterpret_cast<uintptr_t>(requests) % 4 == 0,
             "sample: the scratch buffer must be 256-byte aligned, the requests 4-byte aligned");
  LS_REQUIRE(scratch_bytes >= ls_sample_scratch_bytes(n, vocab), "sample: %ld bytes of scratch, %ld are needed",
             scratch_bytes, ls_sample_scratch_bytes(n, vocab));
  SampleScratch sc;
  char* at = reinterpret_cast<char*>(scratch);
  auto take = [&](size_t bytes) LS_INLINED { char* here = at; at += align_up(bytes); return here; };
  sc.weights = reinterpret_cast<double*>(take((size_t)n * vocab * sizeof(double)));
  sc.keys = reinterpret_cast<unsigned int*>(take((size_t)n * vocab * sizeof(unsigned int)));
  sc.part_max = reinterpret_cast<float*>(take((size_t)n * kChunks * sizeof(float)));
  sc.part_sum = reinterpret_cast<double*>(take((size_t)n * kChunks * sizeof(double)));
  sc.part_level = reinterpret_cast<double*>(take((size_t)2 * n * kChunks * 16 * sizeof(double)));
  sc.state = reinterpret_cast<SearchState*>(take((size_t)4 * n * sizeof(SearchState)));
  sc.tie_count = reinterpret_cast<int*>(take((size_t)n * kChunks * sizeof(int)));
  sc.tie_weight = reinterpret_cast<double*>(take((size_t)n * kChunks * sizeof(double)));
  sc.found = reinterpret_cast<Found*>(take((size_t)2 * n * sizeof(Found)));
  const SampleRow* rows = reinterpret_cast<const SampleRow*>(requests);
  // A row's cut is the same in every call.  Few rows get a workgroup a chunk (a row alone would keep one CU
  // busy); with many rows a workgroup walks several chunks of its row, so that the launch has some
  // LS_SAMPLE_WORKGROUPS_A_CU workgroups a CU instead of thousands of short ones.
  sc.chunks = kChunks;
  if (LS_MUTANT_HOST(kMutantSampleChunksByRows)) sc.chunks = std::max(2, std::min(kChunks, 1024 / n));  // the mutant: a cut that depends on the rows of the call
  const int chunk_len = (vocab + sc.chunks - 1) / sc.chunks;
  const int per_row = std::max(2, std::min(sc.chunks, LS_SAMPLE_WORKGROUPS_A_CU * compute_units() / n));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(per_row, n), block(kSampleThreads);
  hipLaunchKernelGGL(sample_max_kernel, grid, block, 0, s, logits, ld, rows, sc, vocab, chunk_len);
  hipLaunchKernelGGL(sample_exp_kernel, grid, block, 0, s, logits, ld, rows, sc, vocab, chunk_len);
  for (int walk = any_nucleus ? 0 : 1; walk < 2; ++walk) {
    for (int level = 0; level < 8; ++level)
      hipLaunchKernelGGL(sample_level_kernel, grid, block, 0, s, rows, sc, n, vocab, chunk_len, walk, level);
    hipLaunchKernelGGL(sample_tie_count_kernel, grid, block, 0, s, rows, sc, n, vocab, chunk_len, walk);
    hipLaunchKernelGGL(sample_tie_pick_kernel, grid, block, 0, s, rows, sc, n, vocab, chunk_len, walk, out, scatter);
  }
  return check_launch("sample");
}
