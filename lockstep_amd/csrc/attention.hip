// Causal attention over the paged cache, one kernel family for prompt
// portions and for decoded tokens, compiled for one head size (LS_HEAD_DIM).
//
// Rows.  For one sequence and one kv head the queries of the step are laid
// out as rows r = i * G + g (i: query index in the step, g: head inside the
// group of G query heads that share the kv head).  A wave owns 16 rows; a
// lane owns one row (lane % 16) and a quarter of its columns.  With one
// decoded token the G heads share one wave and each key is read once.
//
// Keys.  Positions are tiled in tiles of kTileKeys anchored at multiples of
// kTileKeys, and in splits of kSplitKeys anchored at multiples of kSplitKeys,
// whatever the step's first position is.  Inside a split the tiles are walked
// in ascending order with the online softmax
//     m' = max(m, rowmax(s)); a = exp(m - m'); p = exp(s - m') (s = -inf if masked, so p = 0);
//     l = l*a + sum(p); acc = acc*a + round(p) . V
// (sum(p): a lane adds its four keys of a 16-key block as (p0+p1)+(p2+p3),
// the eight blocks in ascending order, then the four lanes of the row)
// and the splits are folded in ascending order with
//     m' = max(M, m); A = exp(M - m'); B = exp(m - m');
//     ACC = ACC*A + acc*B; L = L*A + l*B
// starting from (0, -1e30, 0); out = ACC / L.  A split that holds no visible
// key for a row (l == 0) is skipped for that row.  A workgroup either walks
// all splits itself and writes the output ("direct"), or handles one split
// and writes (acc, m, l) for the combine kernel, which runs the same fold.
// Both give the same bits, so the choice is free; it is made on the host.
//
// A row's result therefore depends on its own query, its own position and
// the cached keys and values below it, and on nothing else in the launch.
//
// Operands come straight from global memory in the MFMA layouts:
//   S^T = K . Q^T      first operand: 16 keys x one chunk of d (key pages
//                      [page][kv head][slot][d]), second: the wave's 16 rows;
//                      a lane ends with keys 4*(lane/16)+{0..3} of its row.
//   O^T = V^T . P^T    first operand: 16 columns of d x keys (value pages are
//                      stored transposed, [page][kv head][d][slot], so four
//                      consecutive keys of one column are one load), second:
//                      the probabilities exactly as S^T left them in the lane.

#include "common.h"

#ifndef LS_HEAD_DIM
#error "compile with -DLS_HEAD_DIM=<head size, a multiple of 16>"
#endif

#ifdef LS_MUTANTS
__device__ int ls_mutants_dev = 0;  // external linkage: the compiler must not assume it stays zero
#endif

namespace ls {

constexpr int D = LS_HEAD_DIM;
#ifndef LS_STAGED_MIN_BLOCKS
#define LS_STAGED_MIN_BLOCKS 1
#endif
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 up to 256");
constexpr int kTileKeys = 128;
constexpr int kSplitKeys = 128;
#ifndef LS_ATTN_RING
#define LS_ATTN_RING 8
#endif
constexpr int kRing = LS_ATTN_RING;  // LDS operand reads kept in flight ahead of the MFMAs
constexpr int kPageWindow = 32;      // tiles whose page ids a workgroup of the streaming kernels holds in LDS at a time
#ifdef LS_ATTN_PROBE
#define PROBE(i) { long long now_ = clock64(); pr_t[i] += now_ - pr_last; pr_last = now_; }
#ifndef LS_ATTN_PROBE_KVH
#define LS_ATTN_PROBE_KVH 0  // the workgroups of this kv head report
#endif
#else
#define PROBE(i)
#endif
constexpr int NB = kTileKeys / 16;  // 16-key blocks per tile
constexpr int DB = D / 16;          // 16-column blocks of the head

struct SeqMeta {
  int q_off, q_len, q_start, kv_len, table_row, reserved[3];
};
// An item of all zeros stands for no work (lists of graph-replayed steps are rounded up with them): a request
// of no rows has no row to load for and none to write, and the kernels need no test of their own for it.
struct AttnItem {  // one workgroup column of the attention launch (32 ints)
  int seq;         // index into SeqMeta
  int row_block;   // row block of the sequence's rows
  int split_begin, split_end;
  int part_base;   // first partial row of the sequence, or -1: direct
  int n_splits;    // splits of the sequence that have a partial
  int split_lo;    // first of them (splits below lie behind the window)
  int pages_here;  // 1: `pages` holds the page ids of the item's one tile (cooperative items of one tile)
  SeqMeta sm;      // a copy of seqs[seq], so that the kernel needs one load to know its work
  int pages[16];   // the block table's entries for the tile split_begin, so that the tile's loads need no second one
};
static_assert(sizeof(AttnItem) == 128, "the host packs 32 ints an item");

// A masked score is minus infinity, so its probability exp(-inf - m) is an
// exact zero without a select; running maxima start at the finite -1e30, so
// "m" never becomes infinite and no difference of infinities can arise.
constexpr float kMasked = -__builtin_huge_valf();

// One 16-byte piece per lane from global memory straight into LDS: the wave's 64 pieces land at
// `lds_wave_base` + 16 * lane, each lane names its own source.  Written as the instruction itself
// (M0 holds the wave's LDS address): after the compiler's own form of it
// (__builtin_amdgcn_global_load_lds) every later LDS read and every barrier waits for all such
// loads in flight, because they might be reading what the loads write, and the loads of the next
// tile could not overlap the work on this one.  The kernels wait for a tile's loads themselves
// (s_waitcnt vmcnt) before the barrier after which the tile is read.
__device__ __forceinline__ void load_to_lds16(const void* src, __attribute__((address_space(3))) void* lds_wave_base) {
  const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)lds_wave_base);
  __asm__ volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(base) : "memory", "m0");
}

// Sixteen bytes into registers by an instruction the compiler does not know to be a load: it places no wait for
// it, so the kernel can keep it in flight across other loads and wait with a count of its own (wait_for_loads,
// which also ties the registers, so that no use moves above the wait).
__device__ __forceinline__ f32x4 load16_unwaited(const void* src) {
  f32x4 r;
  __asm__ volatile("global_load_dwordx4 %0, %1, off" : "=&v"(r) : "v"(src) : "memory");
  return r;
}
template <int YOUNGER>  // loads issued after those that are waited for (loads complete in the order of their issue)
__device__ __forceinline__ void wait_for_loads(f32x4& a, f32x4& b, f32x4& c, f32x4& d, f32x4& e, f32x4& f, f32x4& g,
                                               f32x4& h) {
  static_assert(YOUNGER >= 0 && YOUNGER <= 63, "the count of a wait has six bits");
  __asm__ volatile("s_waitcnt vmcnt(%8)"
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h)
                   : "n"(YOUNGER)
                   : "memory");
}

// A workgroup barrier that makes the waves' own LDS writes visible and nothing else.  __syncthreads() also
// waits for every load that is still writing into LDS (global_load_lds), which would end the overlap of the
// next tile's loads with the work on this one; where a tile has to be complete, the kernel waits for its own
// loads explicitly (s_waitcnt vmcnt) before the barrier.
__device__ __forceinline__ void lds_barrier() { __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Which key of a tile row r (0..15) of the score block kb stands for.  The score MFMA leaves a lane with rows
// 4g..4g+3 of each 16-key block, and the value MFMA of two such blocks (bfloat16: 32 keys an atom) wants the
// lane's eight probabilities to belong to the eight keys of its value operand.  With the rows of a pair of
// blocks dealt as 0-3, 8-11, 16-19, 24-27 | 4-7, 12-15, 20-23, 28-31 those are the consecutive keys
// 8g..8g+7 of the pair: one 16-byte read of the value tile instead of two of 8 bytes.  float32 atoms take 4 keys
// a lane, which are consecutive anyway.  Every kernel deals the keys through this function, so the sums of the
// probabilities and the products run over the keys in one and the same order everywhere.
template <typename T>
__device__ __forceinline__ constexpr int key_of_row(int kb, int r) {
  return sizeof(T) == 2 ? 32 * (kb >> 1) + 8 * (r >> 2) + 4 * (kb & 1) + (r & 3) : 16 * kb + r;
}
// The rotation of a key row's 16-byte pieces in the LDS tile: the sixteen rows that a score block reads
// together start in sixteen different slots.
template <typename T>
__device__ __forceinline__ constexpr int row_rotation(int row) {
  return sizeof(T) == 2 ? (row & 3) + 4 * ((row >> 3) & 3) : row;
}

// Keep elements n_lo <= e < n_hi of a vector of VEC consecutive keys, zero the others.
__device__ __forceinline__ bf16x8 mask_keys(bf16x8 v, int n_lo, int n_hi) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  u32x4 w = __builtin_bit_cast(u32x4, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned lo = (2 * i >= n_lo && 2 * i < n_hi) ? 0x0000FFFFu : 0u;
    const unsigned hi = (2 * i + 1 >= n_lo && 2 * i + 1 < n_hi) ? 0xFFFF0000u : 0u;
    w[i] = w[i] & (lo | hi);
  }
  return __builtin_bit_cast(bf16x8, w);
}
__device__ __forceinline__ f32x4 mask_keys(f32x4 v, int n_lo, int n_hi) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (e >= n_lo && e < n_hi) ? v[e] : 0.f;
  return v;
}

// All bits set in every element (the operand of mask_keys that turns it into a mask), and the bitwise AND.
template <typename T> __device__ __forceinline__ typename Atom<T>::vec_t ones_vec();
template <> __device__ __forceinline__ bf16x8 ones_vec<bf16_t>() {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  return __builtin_bit_cast(bf16x8, u32x4{0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu});
}
template <> __device__ __forceinline__ f32x4 ones_vec<float>() {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  return __builtin_bit_cast(f32x4, u32x4{0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu});
}
__device__ __forceinline__ bf16x8 and_vec(bf16x8 a, bf16x8 b) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  return __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, a) & __builtin_bit_cast(u32x4, b));
}
__device__ __forceinline__ f32x4 and_vec(f32x4 a, f32x4 b) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  return __builtin_bit_cast(f32x4, __builtin_bit_cast(u32x4, a) & __builtin_bit_cast(u32x4, b));
}

struct RowState {
  f32x4 acc[DB];
  float m, l;
  __device__ __forceinline__ void reset() {
#pragma unroll
    for (int b = 0; b < DB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    m = kNegSentinel;
    l = 0.f;
  }
};

// Fold one split's (acc, m, l) into the running state; the same code runs in
// the attention kernel and in the combine kernel.
template <typename T>
__device__ __forceinline__ void fold_split(RowState& run, const f32x4 (&acc)[DB], float m, float l) {
  if (!(l > 0.f)) return;
  const float m_new = fmaxf(run.m, m);
  const float a = softmax_exp<T>(run.m - m_new);
  const float b = softmax_exp<T>(m - m_new);
#pragma unroll
  for (int blk = 0; blk < DB; ++blk)
#pragma unroll
    for (int e = 0; e < 4; ++e) run.acc[blk][e] = run.acc[blk][e] * a + acc[blk][e] * b;
  run.l = run.l * a + l * b;
  run.m = m_new;
}

template <typename T>
__device__ __forceinline__ void store_output(const RowState& run, T* __restrict__ dst, int g) {
  // dst: start of this row's head in the output; lane writes columns blk*16 + 4g + {0..3}
#pragma unroll
  for (int blk = 0; blk < DB; ++blk) {
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = run.l > 0.f ? run.acc[blk][e] / run.l : 0.f;
    T* p = dst + blk * 16 + 4 * g;
    if (sizeof(T) == 2) {
      bf16x4 v;
      v[0] = (bf16_t)o[0]; v[1] = (bf16_t)o[1]; v[2] = (bf16_t)o[2]; v[3] = (bf16_t)o[3];
      *reinterpret_cast<bf16x4*>(p) = v;
    } else {
      *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
    }
  }
}

// Variant 1, "direct": every wave loads its operands straight from global
// memory.  Needs no LDS, so it takes every head size in both precisions; it
// is the fallback where the staged kernel's tiles do not fit into LDS.
template <typename T>
__global__ __launch_bounds__(256) void attention_direct_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int nkv,
    int page_size, const int* __restrict__ table, int table_stride, const SeqMeta* __restrict__ seqs,
    const AttnItem* __restrict__ items, T* __restrict__ out, long ldo, float* __restrict__ part_acc,
    float* __restrict__ part_ml, int G, float scale, int window) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int NC = (D + A::KCHUNK - 1) / A::KCHUNK;  // chunks over the head

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const AttnItem item = items[blockIdx.x];
  const SeqMeta sm = item.sm;
  const int kvh = blockIdx.y;
  const int rows_total = sm.q_len * G;
  const int r0 = item.row_block * 64 + wave * 16;
  if (r0 >= rows_total) return;

  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int r = r0 + row16;
  const bool row_ok = r < rows_total;
  const int qi = row_ok ? r / G : 0;
  const int head = kvh * G + (row_ok ? r % G : 0);
  const int q_pos = sm.q_start + qi;
  // this row sees the keys key_lo <= key <= key_hi (none if the row does not exist)
  const int key_hi = row_ok ? q_pos : -1;
  const int key_lo = window > 0 ? q_pos - window + 1 : 0;
  const int wave_first_pos = sm.q_start + r0 / G;
  const int wave_last_pos = sm.q_start + min(r0 + 15, rows_total - 1) / G;
  const int lo_valid = window > 0 ? max(0, sm.q_start - window + 1) : 0;
  const int* __restrict__ tbl = table + (long)sm.table_row * table_stride;
  const bool direct = item.part_base < 0;

  vec_t qv[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c)
    qv[c] = load_vec<T>(q + (long)head * D, sm.q_off + qi, c * A::KCHUNK + g * A::VEC, D, ldq, row_ok, true);

  RowState run;
  run.reset();

  for (int split = item.split_begin; split < item.split_end; ++split) {
    const int s_begin = split * kSplitKeys;
    const int s_end = min(s_begin + kSplitKeys, sm.kv_len);
    RowState cur;
    cur.reset();

    for (int t0 = s_begin; t0 < s_end && t0 <= wave_last_pos; t0 += kTileKeys) {
      if (window > 0 && t0 + kTileKeys <= wave_first_pos - window + 1) continue;  // behind every row's window

      // ---- S^T = K . Q^T ---------------------------------------------------
      f32x4 s[NB];
#pragma unroll
      for (int kb = 0; kb < NB; ++kb) {
        s[kb] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int key = t0 + key_of_row<T>(kb, row16);
        bool key_ok = key < sm.kv_len && key >= lo_valid && key <= wave_last_pos;
        long page = key_ok ? tbl[key / page_size] : -1;
        key_ok = key_ok && page >= 0;
        const T* krow = k_pages + (key_ok ? ((page * nkv + kvh) * page_size + key % page_size) * D : 0);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          vec_t kv = load_vec<T>(krow, 0, c * A::KCHUNK + g * A::VEC, D, 0, key_ok, true);
          A::mma(s[kb], kv, qv[c]);
        }
      }

      // ---- scale, mask, online softmax --------------------------------------
      // lane holds keys t0 + kb*16 + 4g + e of its row
      // uniform: every key of the tile is visible to every row of the wave (no mask needed)
      const bool all_visible = t0 + kTileKeys - 1 <= wave_first_pos && r0 + 15 < rows_total &&
                               (window <= 0 || wave_last_pos - t0 < window);
      float tile_max = kNegSentinel;
      if (all_visible) {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s[kb][e] = s[kb][e] * scale;
            tile_max = fmaxf(tile_max, s[kb][e]);
          }
      } else {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int key = t0 + key_of_row<T>(kb, 4 * g + e);
            const float v = ((key <= key_hi) & (key >= key_lo)) ? s[kb][e] * scale : kMasked;
            s[kb][e] = v;
            tile_max = fmaxf(tile_max, v);
          }
      }
      tile_max = quad16_max(tile_max);
      const float m_new = fmaxf(cur.m, tile_max);
      const float alpha = softmax_exp<T>(cur.m - m_new);
      float p_sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < NB; ++kb) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[kb][e] = softmax_exp<T>(s[kb][e] - m_new);  // masked: exp(-inf) = 0
        p_sum = p_sum + ((s[kb][0] + s[kb][1]) + (s[kb][2] + s[kb][3]));
      }
      p_sum = quad16_sum(p_sum);
      cur.l = cur.l * alpha + p_sum;
      cur.m = m_new;
#pragma unroll
      for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int e = 0; e < 4; ++e) cur.acc[blk][e] = cur.acc[blk][e] * alpha;

      // ---- O^T += V^T . P^T --------------------------------------------------
      // one atom covers KB16 blocks of 16 keys: bf16 two (8 keys per lane), f32 one (4 keys per lane)
      constexpr int KB16 = A::VEC / 4;
#pragma unroll
      for (int kb = 0; kb < NB; kb += KB16) {
        vec_t pv;
        long vbase[KB16];
        int vkey[KB16];
#pragma unroll
        for (int h = 0; h < KB16; ++h) {
#pragma unroll
          for (int e = 0; e < 4; ++e) pv[h * 4 + e] = from_f32<T>(s[kb + h][e]);
          const int key = t0 + key_of_row<T>(kb + h, 4 * g);
          vkey[h] = key;
          const bool any = key < sm.kv_len && key + 3 >= lo_valid;
          const long page = any ? tbl[key / page_size] : -1;
          vbase[h] = page >= 0 ? ((page * nkv + kvh) * D) * (long)page_size + key % page_size : -1;
        }
#pragma unroll
        for (int blk = 0; blk < DB; ++blk) {
          vec_t vv = A::zero();
#pragma unroll
          for (int h = 0; h < KB16; ++h) {
            if (vbase[h] >= 0) {
              const T* vp = v_pages + vbase[h] + (long)(blk * 16 + row16) * page_size;
              if (sizeof(T) == 2) {
                bf16x4 four = *reinterpret_cast<const bf16x4*>(vp);
#pragma unroll
                for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
              } else {
                f32x4 four = *reinterpret_cast<const f32x4*>(vp);
#pragma unroll
                for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
              }
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (vkey[h] + e >= sm.kv_len || vkey[h] + e < lo_valid) vv[h * 4 + e] = 0;
            }
          }
          A::mma(cur.acc[blk], vv, pv);
        }
      }
    }

    if (direct) {
      fold_split<T>(run, cur.acc, cur.m, cur.l);
    } else if (row_ok) {
      const long pr = item.part_base + ((long)kvh * rows_total + r) * item.n_splits + (split - item.split_lo);
      float* pa = part_acc + pr * D;
#pragma unroll
      for (int blk = 0; blk < DB; ++blk) *reinterpret_cast<f32x4*>(pa + blk * 16 + 4 * g) = cur.acc[blk];
      if (g == 0) {
        part_ml[pr * 2] = cur.m;
        part_ml[pr * 2 + 1] = cur.l;
      }
    }
  }

  if (direct && row_ok) store_output<T>(run, out + (long)(sm.q_off + qi) * ldo + (long)head * D, g);
}


// Variant 2, "staged": the four waves of a workgroup load each 128-key tile of
// K and of V^T once, with wide coalesced loads, into LDS; every wave then
// takes its MFMA operands from there.  With one decoded token per request
// only the first wave has rows, but all four still fetch, so one workgroup
// keeps 64 KB of loads in flight.  The next tile's global loads are issued
// before the current tile is multiplied.  The arithmetic is the same as in
// the direct variant, instruction for instruction, so both give the same bits.
//
// LDS layout: K tile [128 keys][D], V tile [D][128 keys], rows unpadded; the
// 16-byte pieces of a row are rotated by the row index so that the 16 rows an
// MFMA operand touches fall into different banks.
template <typename T, bool PREFETCH>
__global__ __launch_bounds__(256, LS_STAGED_MIN_BLOCKS) void attention_staged_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int nkv,
    int page_size, int page_shift, const int* __restrict__ table, int table_stride,
    const SeqMeta* __restrict__ seqs, const AttnItem* __restrict__ items, T* __restrict__ out, long ldo,
    float* __restrict__ part_acc, float* __restrict__ part_ml, int G, float scale, int window) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int SZ = sizeof(T);
  constexpr int NC = (D + A::KCHUNK - 1) / A::KCHUNK;
  constexpr int KROW = D * SZ;              // bytes of one key row
  constexpr int KPIECES = KROW / 16;        // 16-byte pieces in it
  constexpr int VROW = kTileKeys * SZ;      // bytes of one column row of the V^T tile
  constexpr int VPIECES = VROW / 16;
  constexpr int TOTAL = kTileKeys * KPIECES;  // pieces in the K tile == pieces in the V tile
  constexpr int PER = (TOTAL + 255) / 256;    // pieces per thread
  constexpr int TILES_PER_SPLIT = kSplitKeys / kTileKeys;
  constexpr int LOG_VEC = (A::VEC == 8) ? 3 : 2;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  unsigned char* k_lds = lds;
  unsigned char* v_lds = lds + kTileKeys * KROW;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const AttnItem item = items[blockIdx.x];
  const SeqMeta sm = item.sm;
  const int kvh = blockIdx.y;
  const int rows_total = sm.q_len * G;
  const int block_r0 = item.row_block * 64;
  if (block_r0 >= rows_total) return;  // uniform for the workgroup
  const int block_first_pos = sm.q_start + block_r0 / G;
  const int block_last_pos = sm.q_start + min(block_r0 + 63, rows_total - 1) / G;

  const int r0 = block_r0 + wave * 16;
  const bool wave_active = r0 < rows_total;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int r = r0 + row16;
  const bool row_ok = r < rows_total;
  const int qi = row_ok ? r / G : 0;
  const int head = kvh * G + (row_ok ? r % G : 0);
  const int q_pos = sm.q_start + qi;
  // this row sees the keys key_lo <= key <= key_hi (none if the row does not exist)
  const int key_hi = row_ok ? q_pos : -1;
  const int key_lo = window > 0 ? q_pos - window + 1 : 0;
  const int wave_first_pos = sm.q_start + min(r0, rows_total - 1) / G;
  const int wave_last_pos = sm.q_start + min(r0 + 15, rows_total - 1) / G;
  const int lo_valid = window > 0 ? max(0, sm.q_start - window + 1) : 0;
  const int* __restrict__ tbl = table + (long)sm.table_row * table_stride;
  const bool direct = item.part_base < 0;
  const int vshift = page_shift - LOG_VEC;  // log2 of the pieces of one column inside a page

  vec_t qv[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c)
    qv[c] = load_vec<T>(q + (long)head * D, sm.q_off + qi, c * A::KCHUNK + g * A::VEC, D, ldq, row_ok, true);

  // tiles this workgroup walks: a contiguous range
  int ti_lo = item.split_begin * TILES_PER_SPLIT;
  if (window > 0) ti_lo = max(ti_lo, max(0, block_first_pos - window + 1) / kTileKeys);
  const int ti_hi = min(item.split_end * TILES_PER_SPLIT, block_last_pos / kTileKeys + 1);

  // Without prefetch the pieces go through registers a few at a time.
  constexpr int GROUP = PREFETCH ? PER : (PER < 4 ? PER : 4);
  // Page ids are looked up one tile ahead of the data they address, so the
  // two dependent loads of a tile do not wait for each other.
  int kpage[PER], vpage[PER];
  auto lookup = [&](int ti) LS_INLINED {
    const int t0 = ti * kTileKeys;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int p = threadIdx.x + 256 * i;
      const int key = t0 + p / KPIECES;
      kpage[i] = tbl[min(key, sm.kv_len - 1) >> page_shift];
      const int q1 = p >> vshift;
      const int key0 = t0 + ((q1 / D) << page_shift) + ((p & ((1 << vshift) - 1)) << LOG_VEC);
      vpage[i] = tbl[min(key0, sm.kv_len - 1) >> page_shift];
    }
  };
  // fetch() only issues loads (from clamped, always valid addresses), so all
  // of a tile's loads are in flight together; stash() zeroes what is not a
  // held key and writes to LDS.
  vec_t kreg[GROUP], vreg[GROUP];
  auto fetch = [&](int ti, int i0) LS_INLINED {
    const int t0 = ti * kTileKeys;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < GROUP; ++j) {
      const int i = i0 + j;
      if (i >= PER) break;
      const int p = threadIdx.x + 256 * i;
      {
        const int key = min(t0 + p / KPIECES, sm.kv_len - 1);
        const int page = max(kpage[i], 0);
        const T* src = k_pages + (((long)page * nkv + kvh) * page_size + (key & (page_size - 1))) * D +
                       (p % KPIECES) * A::VEC;
        kreg[j] = *reinterpret_cast<const vec_t*>(src);
      }
      {
        const int q1 = p >> vshift;
        const int kp = p & ((1 << vshift) - 1);
        const int page = max(vpage[i], 0);
        const T* src = v_pages + ((((long)page * nkv + kvh) * D + q1 % D) << page_shift) + (kp << LOG_VEC);
        vreg[j] = *reinterpret_cast<const vec_t*>(src);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // page ids of the tile whose data is in kreg/vreg (fetch() ran with them)
  int kpage_held[PER], vpage_held[PER];
  auto hold_pages = [&]() LS_INLINED {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      kpage_held[i] = kpage[i];
      vpage_held[i] = vpage[i];
    }
  };
  auto stash = [&](int ti, int i0) LS_INLINED {
    const int t0 = ti * kTileKeys;
#pragma unroll
    for (int j = 0; j < GROUP; ++j) {
      const int i = i0 + j;
      if (i >= PER) break;
      const int p = threadIdx.x + 256 * i;
      const int kt = p / KPIECES;
      const int piece = p % KPIECES;
      const int key = t0 + kt;
      const bool k_ok = key < sm.kv_len && key >= lo_valid && kpage_held[i] >= 0;
      *reinterpret_cast<vec_t*>(k_lds + kt * KROW + ((piece + row_rotation<T>(kt)) % KPIECES) * 16) =
          k_ok ? kreg[j] : A::zero();
      const int q1 = p >> vshift;
      const int kp = p & ((1 << vshift) - 1);
      const int pg = q1 / D;
      const int d = q1 % D;
      const int key0 = t0 + (pg << page_shift) + (kp << LOG_VEC);
      const int n_hi = vpage_held[i] >= 0 ? sm.kv_len - key0 : 0;
      const int vpiece = (pg << vshift) + kp;
      *reinterpret_cast<vec_t*>(v_lds + d * VROW + ((vpiece + d) % VPIECES) * 16) =
          mask_keys(vreg[j], lo_valid - key0, n_hi);
    }
  };

  RowState run, cur;
  run.reset();
  cur.reset();

  if (ti_lo < ti_hi) lookup(ti_lo);
  if (PREFETCH && ti_lo < ti_hi) {
    fetch(ti_lo, 0);
    hold_pages();
    if (ti_lo + 1 < ti_hi) lookup(ti_lo + 1);
  }
#ifdef LS_ATTN_PROBE
  long long pr_t[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  long long pr_last = clock64();
  const long long pr_begin = pr_last;
#endif
  for (int ti = ti_lo; ti < ti_hi; ++ti) {
    const int t0 = ti * kTileKeys;
    __syncthreads();  // the previous tile has been read by every wave
    PROBE(0)
    if (PREFETCH) {
      stash(ti, 0);
    } else {
      hold_pages();
      for (int i0 = 0; i0 < PER; i0 += GROUP) {
        fetch(ti, i0);
        stash(ti, i0);
      }
      if (ti + 1 < ti_hi) lookup(ti + 1);
    }
    PROBE(1)
    __syncthreads();
    PROBE(2)
    if (PREFETCH && ti + 1 < ti_hi) {
      fetch(ti + 1, 0);
      hold_pages();
      if (ti + 2 < ti_hi) lookup(ti + 2);
    }
    PROBE(3)

    const bool mine = wave_active && t0 <= wave_last_pos &&
                      !(window > 0 && t0 + kTileKeys <= wave_first_pos - window + 1);
    if (mine) {
      // ---- S^T = K . Q^T ---------------------------------------------------
      // Operands come from LDS through a ring of registers, read RING products
      // ahead of the MFMA that uses them, so the reads' latency overlaps the
      // matrix work.  The order of the products of one accumulator is unchanged.
      f32x4 s[NB];
      {
        constexpr int NS = NB * NC;
        constexpr int RING = NS < kRing ? NS : kRing;
        auto k_read = [&](int idx) LS_INLINED -> vec_t {
          const int row = key_of_row<T>(idx / NC, row16);
          const int piece = (idx % NC) * 4 + g;
          const int pc = (4 * NC == KPIECES) ? piece : min(piece, KPIECES - 1);
          vec_t kv = *reinterpret_cast<const vec_t*>(k_lds + row * KROW + ((pc + row_rotation<T>(row)) % KPIECES) * 16);
          if (4 * NC != KPIECES) kv = piece < KPIECES ? kv : A::zero();
          return kv;
        };
        vec_t ring[RING];
#pragma unroll
        for (int i = 0; i < RING; ++i) ring[i] = k_read(i);
#pragma unroll
        for (int idx = 0; idx < NS; ++idx) {
          if (idx % NC == 0) s[idx / NC] = f32x4{0.f, 0.f, 0.f, 0.f};
          A::mma(s[idx / NC], ring[idx % RING], qv[idx % NC]);
          if (idx + RING < NS) ring[idx % RING] = k_read(idx + RING);
        }
      }
      PROBE(4)
      // ---- scale, mask, online softmax --------------------------------------
      // uniform: every key of the tile is visible to every row of the wave (no mask needed)
      const bool all_visible = t0 + kTileKeys - 1 <= wave_first_pos && r0 + 15 < rows_total &&
                               (window <= 0 || wave_last_pos - t0 < window);
      float tile_max = kNegSentinel;
      if (all_visible) {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s[kb][e] = s[kb][e] * scale;
            tile_max = fmaxf(tile_max, s[kb][e]);
          }
      } else {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int key = t0 + key_of_row<T>(kb, 4 * g + e);
            const float v = ((key <= key_hi) & (key >= key_lo)) ? s[kb][e] * scale : kMasked;
            s[kb][e] = v;
            tile_max = fmaxf(tile_max, v);
          }
      }
      tile_max = quad16_max(tile_max);
      const float m_new = fmaxf(cur.m, tile_max);
      const float alpha = softmax_exp<T>(cur.m - m_new);
      float p_sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < NB; ++kb) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[kb][e] = softmax_exp<T>(s[kb][e] - m_new);  // masked: exp(-inf) = 0
        p_sum = p_sum + ((s[kb][0] + s[kb][1]) + (s[kb][2] + s[kb][3]));
      }
      p_sum = quad16_sum(p_sum);
      cur.l = cur.l * alpha + p_sum;
      cur.m = m_new;
#pragma unroll
      for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int e = 0; e < 4; ++e) cur.acc[blk][e] = cur.acc[blk][e] * alpha;
      PROBE(5)
      // ---- O^T += V^T . P^T --------------------------------------------------
      constexpr int KB16 = A::VEC / 4;
      {
        constexpr int NP = (NB / KB16) * DB;
        constexpr int RING = NP < kRing ? NP : kRing;
        auto v_read = [&](int idx) LS_INLINED -> vec_t {
          const int kb = (idx / DB) * KB16;
          const int d = (idx % DB) * 16 + row16;
          vec_t vv;
#pragma unroll
          for (int h = 0; h < KB16; ++h) {
            const int byte = key_of_row<T>(kb + h, 4 * g) * SZ;  // offset of the lane's four keys in the column row
            const unsigned char* src = v_lds + d * VROW + (((byte >> 4) + d) % VPIECES) * 16 + (byte & 15);
            if (SZ == 2) {
              bf16x4 four = *reinterpret_cast<const bf16x4*>(src);
#pragma unroll
              for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
            } else {
              f32x4 four = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
              for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
            }
          }
          return vv;
        };
        vec_t ring[RING];
#pragma unroll
        for (int i = 0; i < RING; ++i) ring[i] = v_read(i);
        vec_t pv;
#pragma unroll
        for (int idx = 0; idx < NP; ++idx) {
          if (idx % DB == 0) {
            const int kb = (idx / DB) * KB16;
#pragma unroll
            for (int h = 0; h < KB16; ++h)
#pragma unroll
              for (int e = 0; e < 4; ++e) pv[h * 4 + e] = from_f32<T>(s[kb + h][e]);
          }
          A::mma(cur.acc[idx % DB], ring[idx % RING], pv);
          if (idx + RING < NP) ring[idx % RING] = v_read(idx + RING);
        }
      }
    }
    PROBE(6)
    if (direct && ((ti + 1) % TILES_PER_SPLIT == 0 || ti + 1 == ti_hi)) {
      fold_split<T>(run, cur.acc, cur.m, cur.l);
      cur.reset();
    }
  }

#ifdef LS_ATTN_PROBE
  if (threadIdx.x == 0 && kvh == 0 && part_ml != nullptr) {
    long long* dst = reinterpret_cast<long long*>(part_ml + (1 << 20)) + blockIdx.x * 10;
    for (int i = 0; i < 8; ++i) dst[i] = pr_t[i];
    dst[8] = clock64() - pr_begin;
    dst[9] = ti_hi - ti_lo;
  }
#endif
  if (!row_ok) return;
  if (direct) {
    store_output<T>(run, out + (long)(sm.q_off + qi) * ldo + (long)head * D, g);
  } else {
    const int split = item.split_begin;
    const long pr = item.part_base + ((long)kvh * rows_total + r) * item.n_splits + (split - item.split_lo);
    float* pa = part_acc + pr * D;
#pragma unroll
    for (int blk = 0; blk < DB; ++blk) *reinterpret_cast<f32x4*>(pa + blk * 16 + 4 * g) = cur.acc[blk];
    if (g == 0) {
      part_ml[pr * 2] = cur.m;
      part_ml[pr * 2 + 1] = cur.l;
    }
  }
}


// Variant 4, "wide": prompt portions.  A workgroup of NW waves owns 16*NW rows
// and walks the key tiles with two LDS buffers.  The tiles go from global
// memory straight into LDS (no registers in between): a load instruction of a
// wave fills 64 consecutive 16-byte pieces of LDS, and each lane chooses the
// source of its piece, so the K tile arrives in the rotated layout of the
// staged kernel and the V tile as [8 or 4 keys][column][16 bytes].  While a
// tile is multiplied the next one is in flight.  Keys outside the held range
// need no zeroing in K (their scores are replaced by -inf), and the V tile of
// a boundary tile is cleaned in LDS before use.  The arithmetic of a row is
// the instruction sequence of the other variants, so the bits are the same.
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void attention_wide_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int nkv,
    int page_size, int page_shift, const int* __restrict__ table, int table_stride,
    const SeqMeta* __restrict__ seqs, const AttnItem* __restrict__ items, T* __restrict__ out, long ldo,
    float* __restrict__ part_acc, float* __restrict__ part_ml, int G, float scale, int window) {
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int SZ = sizeof(T);
  constexpr int NT = 64 * NW;
  constexpr int ROWS = 16 * NW;
  constexpr int VEC = A::VEC;
  constexpr int NC = (D + A::KCHUNK - 1) / A::KCHUNK;
  constexpr int KROW = D * SZ;
  constexpr int KPIECES = KROW / 16;
  constexpr int TOTAL = kTileKeys * KPIECES;  // pieces of the K tile == pieces of the V tile
  constexpr int PER = (TOTAL + NT - 1) / NT;
  constexpr int TILE_BYTES = TOTAL * 16;
  constexpr int BUF_BYTES = 2 * TILE_BYTES;
  constexpr int TILES_PER_SPLIT = kSplitKeys / kTileKeys;
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int* tile_pages = reinterpret_cast<int*>(lds + 2 * BUF_BYTES);  // [kPageWindow][16]

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const AttnItem item = items[blockIdx.x];
  const SeqMeta sm = item.sm;
  const int kvh = blockIdx.y;
  const int rows_total = sm.q_len * G;
  const int block_r0 = item.row_block * ROWS;
  if (block_r0 >= rows_total) return;  // uniform for the workgroup
  const int block_first_pos = sm.q_start + block_r0 / G;
  const int block_last_pos = sm.q_start + min(block_r0 + ROWS - 1, rows_total - 1) / G;

  const int r0 = block_r0 + wave * 16;
  const bool wave_active = r0 < rows_total;
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int r = r0 + row16;
  const bool row_ok = r < rows_total;
  const int qi = row_ok ? r / G : 0;
  const int head = kvh * G + (row_ok ? r % G : 0);
  const int q_pos = sm.q_start + qi;
  const int key_hi = row_ok ? q_pos : -1;
  const int key_lo = window > 0 ? q_pos - window + 1 : 0;
  const int wave_first_pos = sm.q_start + min(r0, rows_total - 1) / G;
  const int wave_last_pos = sm.q_start + min(r0 + 15, rows_total - 1) / G;
  const int lo_valid = window > 0 ? max(0, sm.q_start - window + 1) : 0;
  const int* __restrict__ tbl = table + (long)sm.table_row * table_stride;
  const bool direct = item.part_base < 0;
  const int pages_per_tile = kTileKeys >> page_shift;

  vec_t qv[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c)
    qv[c] = load_vec<T>(q + (long)head * D, sm.q_off + qi, c * A::KCHUNK + g * VEC, D, ldq, row_ok, true);

  int ti_lo = item.split_begin * TILES_PER_SPLIT;
  if (window > 0) ti_lo = max(ti_lo, max(0, block_first_pos - window + 1) / kTileKeys);
  const int ti_hi = min(item.split_end * TILES_PER_SPLIT, block_last_pos / kTileKeys + 1);

  // The page ids of kPageWindow tiles at a time go into LDS, by ordinary loads, while no tile load is in
  // flight (the compiler's waits for ordinary loads do not know of the tile loads and would wait for them too).
  auto fill_pages = [&](int first_tile) LS_INLINED {
    for (int idx = threadIdx.x; idx < kPageWindow * 16; idx += NT) {
      const int t = first_tile + idx / 16;
      const int pg = idx % 16;
      if (t < ti_hi && pg < pages_per_tile) {
        const int key = min(t * kTileKeys + (pg << page_shift), sm.kv_len - 1);
        tile_pages[idx] = tbl[key >> page_shift];
      }
    }
  };
  auto window_start = [&](int ti) LS_INLINED -> bool { return (ti - ti_lo) % kPageWindow == 0; };  // tile ti opens a window of ids
  // Start the loads of a tile into its buffer.  What does not depend on the
  // tile is computed once: the offset of each of the thread's pieces inside
  // its page.  Keys past the request's end need no clamp of their own: the
  // page id of their page is that of the last held page (fill_pages clamps),
  // so the loads stay inside the cache, and what they bring is masked.
  const long page_stride = (long)nkv * page_size * D;  // elements of one page, K or V
  int k_off[PER], v_off[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int p = i * NT + (int)threadIdx.x;
    const int row = p / KPIECES;
    const int slot = p % KPIECES;
    const int piece = (slot - row_rotation<T>(row) % KPIECES + KPIECES) % KPIECES;
    k_off[i] = (kvh * page_size + (row & (page_size - 1))) * D + piece * VEC;
    const int c = p / D;
    const int d = p % D;
    v_off[i] = ((kvh * D + d) << page_shift) + ((c * VEC) & (page_size - 1));
  }
  auto issue = [&](int ti) LS_INLINED {
    const int* pages = tile_pages + ((ti - ti_lo) % kPageWindow) * 16;
    unsigned char* k_buf = lds + (ti & 1) * BUF_BYTES;
    unsigned char* v_buf = k_buf + TILE_BYTES;
    int k_page[PER], v_page[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {  // all page ids first: their LDS reads overlap
      const int p = i * NT + (int)threadIdx.x;
      k_page[i] = pages[min((p / KPIECES) >> page_shift, 15)];
      v_page[i] = pages[min(((p / D) * VEC) >> page_shift, 15)];
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      if (PER * NT != TOTAL && i * NT + wave * 64 >= TOTAL) break;  // uniform for the wave
      const T* k_src = k_pages + (long)max(k_page[i], 0) * page_stride + k_off[i];
      load_to_lds16(k_src, (lptr_t)(k_buf + (i * NT + wave * 64) * 16));
      const T* v_src = v_pages + (long)max(v_page[i], 0) * page_stride + v_off[i];
      load_to_lds16(v_src, (lptr_t)(v_buf + (i * NT + wave * 64) * 16));
    }
  };

  RowState run, cur;
  run.reset();
  cur.reset();

  if (ti_lo < ti_hi) {
    fill_pages(ti_lo);
    __syncthreads();
    issue(ti_lo);
  }
#ifdef LS_ATTN_PROBE
  long long pr_t[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  long long pr_last = clock64();
  const long long pr_begin = pr_last;
#endif
#pragma unroll
  for (int c = 0; c < NC; ++c) __asm__ volatile("" ::"v"(qv[c]));  // the query rows are awaited here, not inside the loop
  for (int ti = ti_lo; ti < ti_hi; ++ti) {
    const int t0 = ti * kTileKeys;
    const unsigned char* k_lds = lds + (ti & 1) * BUF_BYTES;
    unsigned char* v_lds = lds + (ti & 1) * BUF_BYTES + TILE_BYTES;
    if (ti != ti_lo && window_start(ti)) {  // nothing is in flight: the previous tile did not request this one
      lds_barrier();
      fill_pages(ti);
      lds_barrier();
      issue(ti);
    }
    __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's pieces of the tile have landed
    PROBE(0)
    lds_barrier();  // the tile is complete, and the other buffer has been read by every wave
    PROBE(1)
    if (t0 + kTileKeys > sm.kv_len || t0 < lo_valid) {  // uniform: clean the values of keys that are not held
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int p = i * NT + (int)threadIdx.x;
        if (PER * NT != TOTAL && p >= TOTAL) break;
        const int key0 = t0 + (p / D) * VEC;
        vec_t* at = reinterpret_cast<vec_t*>(v_lds + p * 16);
        *at = mask_keys(*at, lo_valid - key0, sm.kv_len - key0);
      }
      lds_barrier();
    }
    if (ti + 1 < ti_hi && !window_start(ti + 1)) issue(ti + 1);  // a tile that opens a window of page ids waits for them

    PROBE(2)
    const bool mine = wave_active && t0 <= wave_last_pos &&
                      !(window > 0 && t0 + kTileKeys <= wave_first_pos - window + 1);
    if (mine) {
      // ---- S^T = K . Q^T ---------------------------------------------------
      f32x4 s[NB];
      {
        constexpr int NS = NB * NC;
        constexpr int RING = NS < kRing ? NS : kRing;
        auto k_read = [&](int idx) LS_INLINED -> vec_t {
          const int row = key_of_row<T>(idx / NC, row16);
          const int piece = (idx % NC) * 4 + g;
          const int pc = (4 * NC == KPIECES) ? piece : min(piece, KPIECES - 1);
          vec_t kv = *reinterpret_cast<const vec_t*>(k_lds + row * KROW + ((pc + row_rotation<T>(row)) % KPIECES) * 16);
          if (4 * NC != KPIECES) kv = piece < KPIECES ? kv : A::zero();
          return kv;
        };
        vec_t ring[RING];
#pragma unroll
        for (int i = 0; i < RING; ++i) ring[i] = k_read(i);
#pragma unroll
        for (int idx = 0; idx < NS; ++idx) {
          if (idx % NC == 0) s[idx / NC] = f32x4{0.f, 0.f, 0.f, 0.f};
          A::mma(s[idx / NC], ring[idx % RING], qv[idx % NC]);
          if (idx + RING < NS) ring[idx % RING] = k_read(idx + RING);
        }
      }
      PROBE(3)
      // ---- scale, mask, online softmax --------------------------------------
      const bool all_visible = t0 + kTileKeys - 1 <= wave_first_pos && r0 + 15 < rows_total &&
                               (window <= 0 || wave_last_pos - t0 < window);
      float tile_max = kNegSentinel;
      if (all_visible) {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s[kb][e] = s[kb][e] * scale;
            tile_max = fmaxf(tile_max, s[kb][e]);
          }
      } else {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int key = t0 + key_of_row<T>(kb, 4 * g + e);
            const float v = ((key <= key_hi) & (key >= key_lo)) ? s[kb][e] * scale : kMasked;
            s[kb][e] = v;
            tile_max = fmaxf(tile_max, v);
          }
      }
      tile_max = quad16_max(tile_max);
      const float m_new = fmaxf(cur.m, tile_max);
      const float alpha = softmax_exp<T>(cur.m - m_new);
      float p_sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < NB; ++kb) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[kb][e] = softmax_exp<T>(s[kb][e] - m_new);  // masked: exp(-inf) = 0
        p_sum = p_sum + ((s[kb][0] + s[kb][1]) + (s[kb][2] + s[kb][3]));
      }
      p_sum = quad16_sum(p_sum);
      cur.l = cur.l * alpha + p_sum;
      cur.m = m_new;
#pragma unroll
      for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int e = 0; e < 4; ++e) cur.acc[blk][e] = cur.acc[blk][e] * alpha;
      PROBE(4)
      // ---- O^T += V^T . P^T --------------------------------------------------
      constexpr int KB16 = VEC / 4;
      {
        constexpr int NP = (NB / KB16) * DB;
        constexpr int RING = NP < kRing ? NP : kRing;
        auto v_read = [&](int idx) LS_INLINED -> vec_t {
          const int kb = (idx / DB) * KB16;
          const int d = (idx % DB) * 16 + row16;
          vec_t vv;
#pragma unroll
          for (int h = 0; h < KB16; ++h) {
            const int key = key_of_row<T>(kb + h, 4 * g);  // the lane's four keys inside the tile
            const unsigned char* src = v_lds + ((key / VEC) * D + d) * 16 + (key % VEC) * SZ;
            if (SZ == 2) {
              bf16x4 four = *reinterpret_cast<const bf16x4*>(src);
#pragma unroll
              for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
            } else {
              f32x4 four = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
              for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
            }
          }
          return vv;
        };
        vec_t ring[RING];
#pragma unroll
        for (int i = 0; i < RING; ++i) ring[i] = v_read(i);
        vec_t pv;
#pragma unroll
        for (int idx = 0; idx < NP; ++idx) {
          if (idx % DB == 0) {
            const int kb = (idx / DB) * KB16;
#pragma unroll
            for (int h = 0; h < KB16; ++h)
#pragma unroll
              for (int e = 0; e < 4; ++e) pv[h * 4 + e] = from_f32<T>(s[kb + h][e]);
          }
          A::mma(cur.acc[idx % DB], ring[idx % RING], pv);
          if (idx + RING < NP) ring[idx % RING] = v_read(idx + RING);
        }
      }
    }
    PROBE(5)
    if (direct && ((ti + 1) % TILES_PER_SPLIT == 0 || ti + 1 == ti_hi)) {
      fold_split<T>(run, cur.acc, cur.m, cur.l);
      cur.reset();
    }
  }

#ifdef LS_ATTN_PROBE
  if ((threadIdx.x == 0 || threadIdx.x == 64 * (NW - 1)) && kvh == 0 && part_ml != nullptr) {
    long long* dst = reinterpret_cast<long long*>(part_ml + (1 << 20)) + (blockIdx.x * 2 + (threadIdx.x ? 1 : 0)) * 10;
    for (int i = 0; i < 8; ++i) dst[i] = pr_t[i];
    dst[8] = clock64() - pr_begin;
    dst[9] = ti_hi - ti_lo;
  }
#endif
  if (!row_ok) return;
  if (direct) {
    store_output<T>(run, out + (long)(sm.q_off + qi) * ldo + (long)head * D, g);
  } else {
    const int split = item.split_begin;
    const long pr = item.part_base + ((long)kvh * rows_total + r) * item.n_splits + (split - item.split_lo);
    float* pa = part_acc + pr * D;
#pragma unroll
    for (int blk = 0; blk < DB; ++blk) *reinterpret_cast<f32x4*>(pa + blk * 16 + 4 * g) = cur.acc[blk];
    if (g == 0) {
      part_ml[pr * 2] = cur.m;
      part_ml[pr * 2 + 1] = cur.l;
    }
  }
}


// Variant 3, "cooperative": for work items with at most 16 rows (one decoded
// token per request and up to 16 query heads per kv head), where the other
// kernels would leave most of their waves idle.  All four waves hold the same
// 16 rows.  Wave w computes the score blocks 2w and 2w+1 of a tile and the
// output columns of the blocks w, w+4, ...; row maxima, per-block sums and
// probabilities meet in LDS.  Every number is produced by the same
// instruction sequence as in the other variants, so the bits are the same.
// The data path is the wide kernel's: the K and V tiles go from global memory
// straight into LDS; with NBUF == 2 the next tile is in flight while the four
// waves work on the current one, with NBUF == 1 (large heads, or two workgroups
// a CU) the K half of the single buffer is refilled as soon as the scores exist
// and the V half once the outputs are updated.
//
// With FUSE the kernel also does what qk_rope_kv_kernel does for a step of
// single decoded tokens: `q` is then the raw fused projection (query heads,
// key heads, value heads in a row); the workgroup normalises and rotates its
// query heads into LDS, and the workgroup whose tiles hold the new position
// does the same for the new key, writes key and value to the cache pages and
// patches them into its LDS tile.  Each head goes through head16_finish, as
// in the stand-alone kernel, so the bits are the same.
template <typename T>
struct DecodeFuse {
  const float* q_weight;   // per-head norm weights or nullptr
  const float* k_weight;
  float eps;
  const float* cos_table;  // [positions][rot / 2] or nullptr
  const float* sin_table;
  int rot;
  int nq;                  // query heads in a row of the projection
  int write_kv;            // 0: the cache already holds this step's keys and values
  T* k_out;                // the cache pages, writable
  T* v_out;
};

template <typename T, int NBUF, bool FUSE, bool SPANS>
__global__ __launch_bounds__(256) void attention_coop_kernel(
    // (the first sixteen words of the arguments are in registers when a wave starts: the ones that the first
    // loads of the kernel need come first; `fz` is `fz_rest` with its four tables taken from here)
    const AttnItem* __restrict__ items, const T* __restrict__ q, long ldq, const float* __restrict__ head_q_weight,
    const float* __restrict__ head_k_weight, const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    int G, int nkv, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int page_size, int page_shift,
    const int* __restrict__ table, int table_stride, const SeqMeta* __restrict__ seqs, T* __restrict__ out, long ldo,
    float* __restrict__ part_acc, float* __restrict__ part_ml, float scale, int window, DecodeFuse<T> fz_rest) {
  DecodeFuse<T> fz = fz_rest;
  fz.q_weight = head_q_weight;
  fz.k_weight = head_k_weight;
  fz.cos_table = cos_table;
  fz.sin_table = sin_table;
  typedef Atom<T> A;
  typedef typename A::vec_t vec_t;
  constexpr int SZ = sizeof(T);
  constexpr int NT = 256;
  constexpr int VEC = A::VEC;
  constexpr int NC = (D + A::KCHUNK - 1) / A::KCHUNK;
  constexpr int KROW = D * SZ;
  constexpr int KPIECES = KROW / 16;
  constexpr int TOTAL = kTileKeys * KPIECES;
  constexpr int PER = (TOTAL + NT - 1) / NT;
  constexpr int TILE_BYTES = TOTAL * 16;
  constexpr int BUF_BYTES = 2 * TILE_BYTES;
  constexpr int TILES_PER_SPLIT = kSplitKeys / kTileKeys;
  constexpr int MYDB = (DB + 3) / 4;  // output blocks of one wave
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int* tile_pages = reinterpret_cast<int*>(lds + NBUF * BUF_BYTES);      // [kPageWindow][16]
  float* wmax = reinterpret_cast<float*>(tile_pages + kPageWindow * 16); // [4][16]
  float* psum = wmax + 64;                                               // [NB][64]
  f32x4* prob = reinterpret_cast<f32x4*>(psum + NB * 64);                // [NB][64]
  T* knew = reinterpret_cast<T*>(prob + NB * 64);                        // FUSE: [D] new key, [D] new value
  T* vnew = knew + D;

#ifdef LS_ATTN_PROBE
  long long pr_t[24];
  for (int i = 0; i < 24; ++i) pr_t[i] = 0;
  long long pr_last = clock64();
  const long long pr_begin = pr_last;
#endif
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  // The item is the same for every lane: its fields go to scalar registers, so that what follows from them
  // (tile range, addresses, branch conditions) is scalar work too.
  AttnItem item;
  {
    const int* src = reinterpret_cast<const int*>(items + blockIdx.x);
    int* dst = reinterpret_cast<int*>(&item);
#pragma unroll
    for (int i = 0; i < 16; ++i) dst[i] = __builtin_amdgcn_readfirstlane(src[i]);
  }
  // the page ids an item of one tile brings, one a thread, requested together with the item itself
  const int own_page = FUSE ? items[blockIdx.x].pages[threadIdx.x & 15] : 0;
  if (FUSE) {
    // every other argument is requested now, while the item is on its way: left to themselves their loads
    // stand where each is first used, each with a wait of its own for memory that no cache holds yet
    __asm__ volatile("" ::"s"(k_pages), "s"(v_pages), "s"(page_size), "s"(page_shift), "s"(part_acc), "s"(part_ml),
                     "s"(scale), "s"(window), "s"(fz.eps), "s"(fz.rot), "s"(fz.nq), "s"(fz.write_kv), "s"(fz.k_out),
                     "s"(fz.v_out), "s"(out), "s"(ldo), "s"(table), "s"(table_stride));
  }
  const SeqMeta sm = item.sm;
  const int kvh = blockIdx.y;
  const int rows_total = sm.q_len * G;  // <= 16, checked on the host
  const int row16 = lane & 15;
  const int g = lane >> 4;
  const int r = row16;
  const bool row_ok = r < rows_total;
  const int qi = row_ok ? r / G : 0;
  const int head = kvh * G + (row_ok ? r % G : 0);
  const int q_pos = sm.q_start + qi;
  const int key_hi = row_ok ? q_pos : -1;
  const int key_lo = window > 0 ? q_pos - window + 1 : 0;
  const int first_pos = sm.q_start;
  const int last_pos = sm.q_start + (rows_total - 1) / G;
  const int lo_valid = window > 0 ? max(0, sm.q_start - window + 1) : 0;
  const int* __restrict__ tbl = table + (long)sm.table_row * table_stride;
  const bool direct = item.part_base < 0;
  const int pages_per_tile = kTileKeys >> page_shift;
  if (sm.kv_len < 0) return;
  PROBE(0)

  vec_t qv[NC];
  if (!FUSE) {
#pragma unroll
    for (int c = 0; c < NC; ++c)
      qv[c] = load_vec<T>(q + (long)head * D, sm.q_off + qi, c * A::KCHUNK + g * VEC, D, ldq, row_ok, true);
  }

  int ti_lo = item.split_begin * TILES_PER_SPLIT;
  if (window > 0) ti_lo = max(ti_lo, max(0, first_pos - window + 1) / kTileKeys);
  const int ti_hi = min(item.split_end * TILES_PER_SPLIT, last_pos / kTileKeys + 1);

  // The page ids of kPageWindow tiles at a time go into LDS, by ordinary loads, while no tile load is in
  // flight (the compiler's waits for ordinary loads do not know of the tile loads and would wait for them too).
  auto fill_pages = [&](int first_tile) LS_INLINED {
    for (int idx = threadIdx.x; idx < kPageWindow * 16; idx += NT) {
      const int t = first_tile + idx / 16;
      const int pg = idx % 16;
      if (t < ti_hi && pg < pages_per_tile) {
        const int key = min(t * kTileKeys + (pg << page_shift), sm.kv_len - 1);
        tile_pages[idx] = tbl[key >> page_shift];
      }
    }
  };
  // (an item that brings its one tile's ids: every wave keeps a copy of its own, so that none waits for another)
  const bool embedded = FUSE && item.pages_here != 0;
  auto pages_of = [&](int ti) LS_INLINED -> const int* {
    return tile_pages + (embedded ? wave : (ti - ti_lo) % kPageWindow) * 16;
  };
  auto window_start = [&](int ti) LS_INLINED -> bool { return (ti - ti_lo) % kPageWindow == 0; };  // tile ti opens a window of ids
  const long page_stride = (long)nkv * page_size * D;  // elements of one page, K or V
  PROBE(16)
  // where a thread's pieces of a tile lie inside their pages (the same for every tile)
  int k_off[PER], v_off[PER];
  auto piece_offsets = [&]() LS_INLINED {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int p = i * NT + (int)threadIdx.x;
      const int row = p / KPIECES;
      const int slot = p % KPIECES;
      const int piece = (slot - row_rotation<T>(row) % KPIECES + KPIECES) % KPIECES;
      k_off[i] = (kvh * page_size + (row & (page_size - 1))) * D + piece * VEC;
      const int c = p / D;
      const int d = p % D;
      v_off[i] = ((kvh * D + d) << page_shift) + ((c * VEC) & (page_size - 1));
    }
  };
  auto issue = [&](int ti) LS_INLINED {
    const int* pages = pages_of(ti);
    unsigned char* k_buf = lds + (NBUF == 2 ? (ti & 1) : 0) * BUF_BYTES;
    unsigned char* v_buf = k_buf + TILE_BYTES;
    int k_page[PER], v_page[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {  // all page ids first: their LDS reads overlap
      const int p = i * NT + (int)threadIdx.x;
      k_page[i] = pages[min((p / KPIECES) >> page_shift, 15)];
      v_page[i] = pages[min(((p / D) * VEC) >> page_shift, 15)];
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      if (PER * NT != TOTAL && i * NT + wave * 64 >= TOTAL) break;  // uniform for the wave
      const T* k_src = k_pages + (long)max(k_page[i], 0) * page_stride + k_off[i];
      load_to_lds16(k_src, (lptr_t)(k_buf + (i * NT + wave * 64) * 16));
      const T* v_src = v_pages + (long)max(v_page[i], 0) * page_stride + v_off[i];
      load_to_lds16(v_src, (lptr_t)(v_buf + (i * NT + wave * 64) * 16));
    }
  };
  // With one buffer the K tile and the V tile are loaded apart: the K tile of the next tile as soon as the
  // scores of this one exist, its V tile once the outputs are updated, so a load is in flight most of the time.
  // Each thread issues exactly PER loads for a K tile and PER for a V tile, in this order for a given tile,
  // which is what the waits below count on (loads complete in the order of their issue).
  static_assert(NBUF == 2 || PER * NT == TOTAL, "the split loads assume whole rounds");
  auto issue_k = [&](int ti) LS_INLINED {
    const int* pages = pages_of(ti);
    int k_page[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) k_page[i] = pages[min(((i * NT + (int)threadIdx.x) / KPIECES) >> page_shift, 15)];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const T* k_src = k_pages + (long)max(k_page[i], 0) * page_stride + k_off[i];
      load_to_lds16(k_src, (lptr_t)(lds + (i * NT + wave * 64) * 16));
    }
  };
  auto issue_v = [&](int ti) LS_INLINED {
    const int* pages = pages_of(ti);
    int v_page[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i)
      v_page[i] = pages[min((((i * NT + (int)threadIdx.x) / D) * VEC) >> page_shift, 15)];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const T* v_src = v_pages + (long)max(v_page[i], 0) * page_stride + v_off[i];
      load_to_lds16(v_src, (lptr_t)(lds + TILE_BYTES + (i * NT + wave * 64) * 16));
    }
  };

  // a wave keeps only its own output blocks: block j of the arrays is column block wave + 4j
  f32x4 cur_acc[MYDB], run_acc[MYDB];
  float cur_m = kNegSentinel, cur_l = 0.f, run_m = kNegSentinel, run_l = 0.f;
#pragma unroll
  for (int j = 0; j < MYDB; ++j) {
    cur_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    run_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // The sums of one split to their place among the partial results (an item may hold several splits).
  auto write_partial = [&](int split, const f32x4 (&acc)[MYDB], float m, float l) LS_INLINED {
    if (!row_ok) return;
    const long pr = item.part_base + ((long)kvh * rows_total + r) * item.n_splits + (split - item.split_lo);
    float* pa = part_acc + pr * D;
#pragma unroll
    for (int j = 0; j < MYDB; ++j) {
      const int blk = wave + 4 * j;
      if (blk < DB) *reinterpret_cast<f32x4*>(pa + blk * 16 + 4 * g) = acc[j];
    }
    if (wave == 0 && g == 0) {
      part_ml[pr * 2] = m;
      part_ml[pr * 2 + 1] = l;
    }
  };

  // FUSE: one new token per request at position q_start; its tile is patched by the workgroup that walks it.
  // The heads to process are numbered vi: the G query heads, then the new key, then the new value;
  // wave w takes vi = w, w + 4, ...  The operands of its first head are loaded before the tile loads start.
  const int p_new = sm.q_start;
  const int tile_new = p_new / kTileKeys;
  const bool owner = FUSE && fz.write_kv && tile_new >= ti_lo && tile_new < ti_hi;
  const int n_vec = owner ? G + 2 : G;
  const T* new_row = q + (long)sm.q_off * ldq;
  const bool rotated = FUSE && fz.cos_table != nullptr;
  // Sixteen lanes a head (head16_finish): the workgroup's sixteen groups take the heads vi = group, group + 16.
  constexpr int PASSES = D > 128 ? 2 : 1;
  const int gl = threadIdx.x & 15;
  // the head a group of sixteen lanes takes: the first four heads go to the first group of each wave, the next
  // four to the second groups, ... (a step has mostly four heads a workgroup: two query heads, the key and the
  // value; in one wave their different branches would run one after the other)
  const int grp = ((threadIdx.x >> 4) & 3) * 4 + (threadIdx.x >> 6);
  long page_new = -1;
  float hx[8 * PASSES] = {};
  HeadFactors<PASSES> hf = {};
  auto head_src = [&](int vi) LS_INLINED -> const T* {
    return new_row + (long)(vi < G ? kvh * G + vi : vi == G ? fz.nq + kvh : fz.nq + nkv + kvh) * D;
  };
  auto head_fetch = [&](int vi) LS_INLINED {
    head16_load_values<T, PASSES>(hx, head_src(vi), D, gl);
    if (vi <= G)
      head16_load_factors<PASSES>(hf, D, vi < G ? fz.q_weight : fz.k_weight, fz.cos_table, fz.sin_table, p_new,
                                  fz.rot, gl);
  };
  T* qrot = reinterpret_cast<T*>(prob);  // FUSE: [16][D] rotated query heads; the exchange buffers are free until the loop
  // norm and rotation of head vi from hx / hf: a query head to qrot, the new key and value to LDS and to the cache
  auto finish_head = [&](int vi) LS_INLINED {
    if (vi < G) {
      head16_finish<T, PASSES>(hx, hf, D, fz.q_weight != nullptr, fz.eps, rotated, fz.rot, gl,
                               [&](int e0, const T (&v)[8]) LS_INLINED { store8<T>(qrot + vi * D + e0, v); });
    } else if (vi == G) {
      head16_finish<T, PASSES>(hx, hf, D, fz.k_weight != nullptr, fz.eps, rotated, fz.rot, gl,
                               [&](int e0, const T (&v)[8]) LS_INLINED { store8<T>(knew + e0, v); });
    } else {
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        const int e0 = 128 * p + 8 * gl;
        if (e0 >= D) continue;
#pragma unroll
        for (int j = 0; j < 8; ++j) vnew[e0 + j] = from_f32<T>(hx[8 * p + j]);
      }
    }
  };
  // The new key and value go from LDS to the cache when the workgroup's tiles are done: a store issued while
  // the tile loads are queued waits behind them, and its wave reaches the next barrier that much later.
  auto write_new_to_cache = [&]() LS_INLINED {
    if (page_new < 0) return;
    const int slot_new = p_new & (page_size - 1);
    T* k_dst = fz.k_out + ((page_new * nkv + kvh) * page_size + slot_new) * D;
    T* v_dst = fz.v_out + ((page_new * nkv + kvh) * D) * page_size + slot_new;
    const int t = (int)threadIdx.x - (NT - 64);  // the key by the last wave, the value by the first ones
    if (t >= 0 && 8 * t < D) {
      T piece[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) piece[j] = knew[8 * t + j];
      store8<T>(k_dst + 8 * t, piece);
    }
    for (int e = threadIdx.x; e < D; e += NT) v_dst[(long)e * page_size] = vnew[e];
  };
  // An item of one tile may bring the tile's page ids itself (embedded): the tile loads then wait for no second
  // round trip.  The head's operands are then requested by loads the compiler does not count (unwaited), ahead
  // of the tile loads, and awaited with a count that leaves the tile loads in flight, so that norm, rotation and
  // cache write run while the tile is on its way.
  PROBE(18)
  // (the ids go to their place in LDS before any unwaited load is issued: the compiler's wait for `own_page`
  // would wait for those as well)
  if (embedded && lane < 16) tile_pages[wave * 16 + lane] = own_page;
  PROBE(19)
  const bool aligned_turn = !rotated || (((fz.rot / 2) & 7) == 0);
  const bool unwaited = embedded && PASSES == 1 && aligned_turn && n_vec <= 16 && 2 * PER <= 63;
  const int e0_head = 8 * gl;                    // the lane's eight elements of a head (PASSES == 1)
  const bool lane_in_head = e0_head < D;
  const bool lane_turns = rotated && e0_head < fz.rot;
  auto issue_tile = [&](int ti) LS_INLINED {
    if (NBUF == 2) {
      issue(ti);
    } else {
      issue_k(ti);
      issue_v(ti);
    }
  };
  constexpr bool CAN_PRIME = NBUF == 2 && 2 * PER <= 63;  // (the wait names the loads of one tile: a 6-bit count)
  bool primed = false;
  if (FUSE && unwaited) {
    if constexpr (PASSES == 1 && 2 * PER <= 63) {  // (what `unwaited` asks for, said to the compiler)
      // Straight-line code from the loads to their wait, every load unconditional: a register that such a load
      // writes must not be copied or merged with another value before the wait (the compiler takes it to be
      // written when the instruction is issued).  Lanes and groups that need no operand load a spare address
      // and drop the result.
      const int vi = min(grp, n_vec - 1);
      const float* spare = reinterpret_cast<const float*>(items + blockIdx.x);  // 128 readable bytes
      const T* src = head_src(vi) + (lane_in_head ? e0_head : 0);
      const float* weight = vi < G ? fz.q_weight : vi == G ? fz.k_weight : nullptr;
      const bool weighted = weight != nullptr && lane_in_head && grp < n_vec;
      const float* w_at = weighted ? weight + e0_head : spare;
      const int half = fz.rot / 2;
      const bool turns = lane_turns && vi <= G;
      const float* c_at = turns ? fz.cos_table + (long)p_new * half + (e0_head < half ? e0_head : e0_head - half) : spare;
      const float* s_at = turns ? fz.sin_table + (long)p_new * half + (e0_head < half ? e0_head : e0_head - half) : spare;
      PROBE(12)
      f32x4 raw_x0 = load16_unwaited(src);
      f32x4 raw_x1 = load16_unwaited(sizeof(T) == 4 ? reinterpret_cast<const float*>(src) + 4 : spare);
      f32x4 raw_w0 = load16_unwaited(w_at);
      f32x4 raw_w1 = load16_unwaited(w_at + 4);
      f32x4 raw_c0 = load16_unwaited(c_at);
      f32x4 raw_c1 = load16_unwaited(c_at + 4);
      f32x4 raw_s0 = load16_unwaited(s_at);
      f32x4 raw_s1 = load16_unwaited(s_at + 4);
      PROBE(13)
      piece_offsets();  // (while the loads are on their way)
      if (owner) page_new = tile_pages[wave * 16 + ((p_new & (kTileKeys - 1)) >> page_shift)];
      PROBE(1)
      // the head's operands: everything but the tile's 2 * PER loads (if the item has a tile at all) has arrived
      // (one wait statement for both cases, so that the registers reach it by one way only and are not moved on
      // the way; without a tile everything is awaited first, and the counted wait finds nothing left)
      if (ti_lo < ti_hi)
        issue_tile(ti_lo);
      else
        __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
      wait_for_loads<2 * PER>(raw_x0, raw_x1, raw_w0, raw_w1, raw_c0, raw_c1, raw_s0, raw_s1);
      PROBE(2)
      if (sizeof(T) == 2) {
        const bf16x8 v = __builtin_bit_cast(bf16x8, raw_x0);
#pragma unroll
        for (int j = 0; j < 8; ++j) hx[j] = lane_in_head ? to_f32(v[j]) : 0.f;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          hx[j] = lane_in_head ? raw_x0[j] : 0.f;
          hx[4 + j] = lane_in_head ? raw_x1[j] : 0.f;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        hf.w[j] = weighted ? raw_w0[j] : 1.f;
        hf.w[4 + j] = weighted ? raw_w1[j] : 1.f;
        hf.c[j] = turns ? raw_c0[j] : 1.f;
        hf.c[4 + j] = turns ? raw_c1[j] : 1.f;
        hf.s[j] = turns ? raw_s0[j] : 0.f;
        hf.s[4 + j] = turns ? raw_s1[j] : 0.f;
      }
    }
  } else {
    piece_offsets();
    if (FUSE) {
      if (owner && !embedded) page_new = tbl[p_new >> page_shift];
      if (grp < n_vec) head_fetch(grp);
    }
    if (!embedded && ti_lo < ti_hi) fill_pages(ti_lo);
    __syncthreads();
    if (embedded && owner) page_new = tile_pages[wave * 16 + ((p_new & (kTileKeys - 1)) >> page_shift)];
    if (FUSE) {
      // The head's operands are awaited here, before the tile loads go out: a wait placed after them would also
      // wait for the tiles (loads complete in the order of their issue, and the compiler does not count the tile
      // loads), and the norm, the rotation and the cache write below would start only when the tiles are in.
#pragma unroll
      for (int i = 0; i < 8 * PASSES; ++i) __asm__ volatile("" ::"v"(hx[i]), "v"(hf.w[i]), "v"(hf.c[i]), "v"(hf.s[i]));
      __asm__ volatile("" ::"v"((int)page_new));
      if (n_vec > 16) {  // more heads than groups of sixteen lanes (fifteen query heads a kv head and more): all of
        finish_head(grp);  // them now, so that no load of a head stands behind the tile loads
        if (grp + 16 < n_vec) {
          head_fetch(grp + 16);
          finish_head(grp + 16);
        }
      }
    }
    PROBE(1)
    if (ti_lo < ti_hi) issue_tile(ti_lo);
    // two buffers: both are free now, so the second tile is requested at once as well and its wait overlaps the
    // first one's (a workgroup of a decode step mostly has two tiles, and a miss takes longer than a tile's work)
    primed = CAN_PRIME && !embedded && ti_lo + 1 < ti_hi && !window_start(ti_lo + 1);
    if (primed) issue(ti_lo + 1);
  }
  PROBE(2)
  if (FUSE) {
    if (n_vec <= 16 && grp < n_vec) finish_head(grp);  // (more heads than groups: done above, before the tile loads)
    PROBE(14)
    lds_barrier();
    PROBE(15)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int col = c * A::KCHUNK + g * VEC;
      qv[c] = (row_ok && col < D) ? *reinterpret_cast<const vec_t*>(qrot + row16 * D + min(col, D - VEC)) : A::zero();
    }
  }
  if (!FUSE) {  // the query rows, loaded from global memory, are awaited here and not inside the loop
#pragma unroll
    for (int c = 0; c < NC; ++c) __asm__ volatile("" ::"v"(qv[c]));
  }
  PROBE(3)
  for (int ti = ti_lo; ti < ti_hi; ++ti) {
    const int t0 = ti * kTileKeys;
    const unsigned char* k_lds = lds + (NBUF == 2 ? (ti & 1) : 0) * BUF_BYTES;
    unsigned char* v_lds = lds + (NBUF == 2 ? (ti & 1) : 0) * BUF_BYTES + TILE_BYTES;
    // the next tile is requested ahead unless it opens a new window of page ids
    const bool ahead = ti + 1 < ti_hi && !window_start(ti + 1);
    if (ti != ti_lo && window_start(ti)) {  // nothing is in flight: the previous tile did not request this one
      lds_barrier();
      fill_pages(ti);
      lds_barrier();
      issue_tile(ti);
    }
    if (NBUF == 2) {
      // this thread's pieces of the tile have landed (loads complete in the order of their issue: behind the
      // first tile only the 2 * PER loads of the second one, and stores, may still be on their way)
      if (primed && ti == ti_lo) {
        if constexpr (CAN_PRIME) __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PER) : "memory");
      } else {
        __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    } else {
      // this thread's pieces of the K tile have landed; its PER loads of the V tile, issued later, may be in flight
      __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(PER) : "memory");
    }
    PROBE(4)
    lds_barrier();  // the tile (one buffer: its K half) is complete (and the other buffer has been read by every wave)
    PROBE(5)
    const bool patch = owner && ti == tile_new;  // the new key and value go into this tile
    const bool clean = t0 + kTileKeys > sm.kv_len || t0 < lo_valid || patch;  // uniform
    if (FUSE && patch) {  // the new key goes into the K tile now; the values are dealt with where they are read
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int p = i * NT + (int)threadIdx.x;
        const int row = p / KPIECES;
        if (t0 + row == p_new) {
          const int piece = (p % KPIECES - row_rotation<T>(row) % KPIECES + KPIECES) % KPIECES;
          *reinterpret_cast<vec_t*>(const_cast<unsigned char*>(k_lds) + p * 16) =
              *reinterpret_cast<const vec_t*>(knew + piece * VEC);
        }
      }
      lds_barrier();
    }
    if (NBUF == 2 && ahead && !(primed && ti == ti_lo)) issue(ti + 1);

    // score blocks 2w and 2w+1
    PROBE(6)
    f32x4 s[2];
    float my_max = kNegSentinel;
    {
      vec_t kop[2][NC];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = key_of_row<T>(2 * wave + j, row16);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int piece = c * 4 + g;
          const int pc = (4 * NC == KPIECES) ? piece : min(piece, KPIECES - 1);
          vec_t kv = *reinterpret_cast<const vec_t*>(k_lds + row * KROW + ((pc + row_rotation<T>(row)) % KPIECES) * 16);
          if (4 * NC != KPIECES) kv = piece < KPIECES ? kv : A::zero();
          kop[j][c] = kv;
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int kb = 2 * wave + j;
        s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c) A::mma(s[j], kop[j][c], qv[c]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = t0 + key_of_row<T>(kb, 4 * g + e);
          const float v = ((key <= key_hi) & (key >= key_lo)) ? s[j][e] * scale : kMasked;
          s[j][e] = v;
          my_max = fmaxf(my_max, v);
        }
      }
    }
    my_max = quad16_max(my_max);
    if (g == 0) wmax[wave * 16 + row16] = my_max;
    PROBE(7)
    lds_barrier();
    PROBE(8)
    if (NBUF == 1 && ahead) issue_k(ti + 1);  // every wave has its scores: the K half of the buffer is free
    const float tile_max = fmaxf(fmaxf(wmax[row16], wmax[16 + row16]), fmaxf(wmax[32 + row16], wmax[48 + row16]));
    const float m_new = fmaxf(cur_m, tile_max);
    const float alpha = softmax_exp<T>(cur_m - m_new);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int kb = 2 * wave + j;
#pragma unroll
      for (int e = 0; e < 4; ++e) s[j][e] = softmax_exp<T>(s[j][e] - m_new);  // masked: exp(-inf) = 0
      psum[kb * 64 + lane] = (s[j][0] + s[j][1]) + (s[j][2] + s[j][3]);
      prob[kb * 64 + lane] = s[j];
    }
    // this wave's value operands do not depend on the probabilities: with two buffers they are read before the
    // barrier; with one buffer the V tile is only now awaited (the K loads of the next tile, issued after it,
    // may stay in flight) and complete for every thread after the barrier
    constexpr int KB16 = VEC / 4;
    constexpr int NPAIR = NB / KB16;
    vec_t vop[NPAIR][MYDB];
    auto read_values = [&]() LS_INLINED {
#pragma unroll
    for (int kp = 0; kp < NPAIR; ++kp)
#pragma unroll
      for (int j = 0; j < MYDB; ++j) {
        const int blk = wave + 4 * j;
        const int d = (blk < DB ? blk : 0) * 16 + row16;
        vec_t vv;
#pragma unroll
        for (int h = 0; h < KB16; ++h) {
          const int key = key_of_row<T>(kp * KB16 + h, 4 * g);
          const unsigned char* src = v_lds + ((key / VEC) * D + d) * 16 + (key % VEC) * SZ;
          if (SZ == 2) {
            bf16x4 four = *reinterpret_cast<const bf16x4*>(src);
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
          } else {
            f32x4 four = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[h * 4 + e] = four[e];
          }
        }
        vop[kp][j] = vv;
      }
    };
    // The values of keys that are not held become zeros and the new token's value takes its place: in the
    // operands as they were read (a lane's VEC values of a column belong to VEC consecutive keys), not in LDS.
    auto fix_values = [&]() LS_INLINED {
#pragma unroll
      for (int kp = 0; kp < NPAIR; ++kp) {
        const int key0 = t0 + key_of_row<T>(kp * KB16, 4 * g);
        const int n_lo = lo_valid - key0, n_hi = sm.kv_len - key0;
        const int first_key = t0 + kp * (16 * KB16), end_key = first_key + 16 * KB16;  // of all lanes together
        const bool has_new = FUSE && patch && p_new >= first_key && p_new < end_key;
        if (end_key <= sm.kv_len && first_key >= lo_valid && !has_new) continue;  // uniform: every key is held
        if ((first_key >= sm.kv_len || end_key <= lo_valid) && !has_new) {        // uniform: none is
#pragma unroll
          for (int j = 0; j < MYDB; ++j) vop[kp][j] = A::zero();
          continue;
        }
        if (n_lo > 0 || n_hi < VEC) {
          // one mask for the lane's VEC keys, used for all of its columns
          const vec_t keep = mask_keys(ones_vec<T>(), n_lo, n_hi);
#pragma unroll
          for (int j = 0; j < MYDB; ++j) vop[kp][j] = and_vec(vop[kp][j], keep);
        }
        if (FUSE && patch && p_new >= key0 && p_new < key0 + VEC) {
#pragma unroll
          for (int j = 0; j < MYDB; ++j) {
            const int blk = wave + 4 * j;
            const T fresh = vnew[(blk < DB ? blk : 0) * 16 + row16];
            vec_t v = vop[kp][j];
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = key0 + e == p_new ? fresh : v[e];
            vop[kp][j] = v;
          }
        }
      }
    };
    if (NBUF == 2) {
      read_values();
      if (clean) fix_values();
    } else if (ahead) {
      __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(PER) : "memory");
    } else {
      __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    PROBE(9)
    lds_barrier();
    PROBE(10)
    if (NBUF == 1) {
      read_values();
      if (clean) fix_values();
    }
    float p_sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < NB; ++kb) p_sum = p_sum + psum[kb * 64 + lane];
    p_sum = quad16_sum(p_sum);
    cur_l = cur_l * alpha + p_sum;
    cur_m = m_new;
#pragma unroll
    for (int j = 0; j < MYDB; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) cur_acc[j][e] = cur_acc[j][e] * alpha;
#pragma unroll
    for (int kp = 0; kp < NPAIR; ++kp) {
      vec_t pv;
#pragma unroll
      for (int h = 0; h < KB16; ++h) {
        const f32x4 four = prob[(kp * KB16 + h) * 64 + lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) pv[h * 4 + e] = from_f32<T>(four[e]);
      }
#pragma unroll
      for (int j = 0; j < MYDB; ++j) {
        if (wave + 4 * j >= DB) continue;
        A::mma(cur_acc[j], vop[kp][j], pv);
      }
    }
    PROBE(11)
    if (SPANS) {
      if (!direct && (ti + 1) % TILES_PER_SPLIT == 0 && ti + 1 < ti_hi) {  // an item of several splits: this one's
        write_partial(ti / TILES_PER_SPLIT, cur_acc, cur_m, cur_l);        // sums go to their place
#pragma unroll
        for (int j = 0; j < MYDB; ++j) cur_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        cur_m = kNegSentinel;
        cur_l = 0.f;
      }
    }
    if (direct && ((ti + 1) % TILES_PER_SPLIT == 0 || ti + 1 == ti_hi)) {
      if (cur_l > 0.f) {  // the fold of fold_split, on this wave's blocks
        const float m_fold = fmaxf(run_m, cur_m);
        const float fa = softmax_exp<T>(run_m - m_fold);
        const float fb = softmax_exp<T>(cur_m - m_fold);
#pragma unroll
        for (int j = 0; j < MYDB; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) run_acc[j][e] = run_acc[j][e] * fa + cur_acc[j][e] * fb;
        run_l = run_l * fa + cur_l * fb;
        run_m = m_fold;
      }
#pragma unroll
      for (int j = 0; j < MYDB; ++j) cur_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      cur_m = kNegSentinel;
      cur_l = 0.f;
    }
    if (NBUF == 1 && ti + 1 < ti_hi) {
      lds_barrier();  // every wave is done with the V half of the buffer
      if (ahead) issue_v(ti + 1);
    }
  }

  if (FUSE && owner) write_new_to_cache();
#ifdef LS_ATTN_PROBE
  if (threadIdx.x == 0 && kvh == LS_ATTN_PROBE_KVH && part_ml != nullptr) {
    long long* dst = reinterpret_cast<long long*>(part_ml + (1 << 20)) + blockIdx.x * 32;
    for (int i = 0; i < 12; ++i) dst[i] = pr_t[i];
    dst[12] = clock64() - pr_begin;
    dst[13] = ti_hi - ti_lo;
    for (int i = 12; i < 24; ++i) dst[i + 4] = pr_t[i];
  }
#endif
  if (!row_ok) return;
  if (direct) {
    T* dst = out + (long)(sm.q_off + qi) * ldo + (long)head * D;
    const float l = run_l;
#pragma unroll
    for (int j = 0; j < MYDB; ++j) {
      const int blk = wave + 4 * j;
      if (blk >= DB) continue;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = l > 0.f ? run_acc[j][e] / l : 0.f;
      T* p = dst + blk * 16 + 4 * g;
      if (SZ == 2) {
        bf16x4 v;
        v[0] = (bf16_t)o[0]; v[1] = (bf16_t)o[1]; v[2] = (bf16_t)o[2]; v[3] = (bf16_t)o[3];
        *reinterpret_cast<bf16x4*>(p) = v;
      } else {
        *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
      }
    }
  } else {
    // the item's splits that hold no tile for these rows (past the request's end, or behind the window)
    // leave empty sums: the fold reads every split's place and skips those
    if (!SPANS) {  // one split an item (checked on the host): its sums, empty if it holds no tile for these rows
      const int split = item.split_begin;
      const long pr = item.part_base + ((long)kvh * rows_total + r) * item.n_splits + (split - item.split_lo);
      float* pa = part_acc + pr * D;
#pragma unroll
      for (int j = 0; j < MYDB; ++j) {
        const int blk = wave + 4 * j;
        if (blk < DB) *reinterpret_cast<f32x4*>(pa + blk * 16 + 4 * g) = cur_acc[j];
      }
      if (wave == 0 && g == 0) {
        part_ml[pr * 2] = cur_m;
        part_ml[pr * 2 + 1] = cur_l;
      }
      return;
    }
    const int first_done = ti_lo / TILES_PER_SPLIT, last_done = (ti_hi - 1) / TILES_PER_SPLIT;
    if (ti_lo < ti_hi) {  // the sums of the last split walked
      write_partial(last_done, cur_acc, cur_m, cur_l);
#pragma unroll
      for (int j = 0; j < MYDB; ++j) cur_acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int split = item.split_begin; split < item.split_end; ++split)
      if (ti_lo >= ti_hi || split < first_done || split > last_done) write_partial(split, cur_acc, kNegSentinel, 0.f);
  }
}

struct CombineItem {  // 8 ints
  int seq, row_block, part_base, n_splits;
  int q_off, q_len;  // of seqs[seq]
  int reserved[2];
};

// The fold of one block of 64 rows of a request: a lane takes a row and a quarter of its columns.
template <typename T>
__device__ __forceinline__ void combine_row_block(const CombineItem& item, int row_block, int kvh,
                                                  const float* __restrict__ part_acc,
                                                  const float* __restrict__ part_ml, T* __restrict__ out, long ldo,
                                                  int G) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int rows_total = item.q_len * G;
  const int r = row_block * 64 + wave * 16 + (lane & 15);
  if (r >= rows_total) return;
  const int g = lane >> 4;
  const int qi = r / G;
  const int head = kvh * G + r % G;

  RowState run;
  run.reset();
  const long pr0 = item.part_base + ((long)kvh * rows_total + r) * item.n_splits;
  // The partial results of several splits are requested together (a request far away has many splits and
  // the fold of each waits for its loads); they are folded in ascending order all the same.
  constexpr int BATCH = DB <= 8 ? 4 : 2;
  if (LS_MUTANT_DEVICE(kMutantReversedFold)) {
    for (int s = item.n_splits - 1; s >= 0; --s) {
      f32x4 acc[DB];
      const long pr = pr0 + s;
#pragma unroll
      for (int blk = 0; blk < DB; ++blk)
        acc[blk] = *reinterpret_cast<const f32x4*>(part_acc + pr * D + blk * 16 + 4 * g);
      fold_split<T>(run, acc, part_ml[pr * 2], part_ml[pr * 2 + 1]);
    }
    store_output<T>(run, out + (long)(item.q_off + qi) * ldo + (long)head * D, g);
    return;
  }
  for (int s0 = 0; s0 < item.n_splits; s0 += BATCH) {
    f32x4 acc[BATCH][DB];
    float m[BATCH], l[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const long pr = pr0 + min(s0 + u, item.n_splits - 1);  // clamped: loaded, not used
#pragma unroll
      for (int blk = 0; blk < DB; ++blk)
        acc[u][blk] = *reinterpret_cast<const f32x4*>(part_acc + pr * D + blk * 16 + 4 * g);
      m[u] = part_ml[pr * 2];
      l[u] = part_ml[pr * 2 + 1];
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u)
      if (s0 + u < item.n_splits) fold_split<T>(run, acc[u], m[u], l[u]);
  }
  store_output<T>(run, out + (long)(item.q_off + qi) * ldo + (long)head * D, g);
}

template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(const SeqMeta* __restrict__ seqs,
                                                      const CombineItem* __restrict__ items,
                                                      const float* __restrict__ part_acc,
                                                      const float* __restrict__ part_ml, T* __restrict__ out,
                                                      long ldo, int G) {
  const CombineItem item = items[blockIdx.x];
  combine_row_block<T>(item, item.row_block, blockIdx.y, part_acc, part_ml, out, ldo, G);
}

// The fold for requests of at most 16 rows a kv head (decoded tokens), where a request far away has dozens
// of splits.  The fold of one split has to wait for the one before, so what counts is how long one fold
// takes and that its operands are there.  All 256 threads bring the partial results of a batch of splits
// into LDS in whole lines (a row's splits lie one after the other), the next batch's loads are in flight
// while this one is folded, and the folding itself is dealt out by elements: a thread owns four
// neighbouring columns of one row (with two rows of 128 columns one wave does all of it, every lane busy,
// a fold is some twenty instructions).  Every element goes through the operations of fold_split in the
// same order: the same bits.
template <typename T>
__global__ __launch_bounds__(256) void combine_few_rows_kernel(const SeqMeta* __restrict__ seqs,
                                                               const CombineItem* __restrict__ items,
                                                               const float* __restrict__ part_acc,
                                                               const float* __restrict__ part_ml,
                                                               T* __restrict__ out, long ldo, int G) {
  constexpr int QUADS = D / 4;                       // groups of four columns in a row
  constexpr int MAXQ = (16 * QUADS + 255) / 256;     // such groups a thread owns at most (16 rows)
  constexpr int STAGE = 6144;                        // floats of sums a buffer holds
  constexpr int ROW_PAD = 4;                         // floats between rows: spreads the rows over the banks
  constexpr int PIECES = STAGE / 4 / 256;            // 16-byte pieces a thread moves per batch
  __shared__ __attribute__((aligned(16))) float stage_acc[2][STAGE];
  __shared__ float stage_ml[2][2 * 512];
  const CombineItem item = items[blockIdx.x];
  const int kvh = blockIdx.y;
  const int rows_total = item.q_len * G;
  if (rows_total <= 0) return;
  if (rows_total > 16) {
    // more rows than this kernel's threads own columns for (the caller promised otherwise): the general
    // fold, block of rows by block of rows -- the same bits, only slower
    for (int block = 0; block * 64 < rows_total; ++block)
      combine_row_block<T>(item, block, kvh, part_acc, part_ml, out, ldo, G);
    return;
  }
  const int n_splits = item.n_splits;
  const long pr_base = item.part_base + (long)kvh * rows_total * n_splits;  // row r, split s: pr_base + r * n_splits + s
  const int owned = rows_total * QUADS;   // groups of four columns to fold

  f32x4 run_acc[MAXQ];
  float run_m[MAXQ], run_l[MAXQ];
  int row_of[MAXQ], quad_of[MAXQ];
#pragma unroll
  for (int q = 0; q < MAXQ; ++q) {
    run_acc[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    run_m[q] = kNegSentinel;
    run_l[q] = 0.f;
    const int it = min(q * 256 + (int)threadIdx.x, owned - 1);
    row_of[q] = it / QUADS;
    quad_of[q] = it - row_of[q] * QUADS;
  }
  // (not under the reversed-fold mutant, whose loop folds by groups of four columns)
  const bool narrow = rows_total * D <= 256 && !LS_MUTANT_DEVICE(kMutantReversedFold);
  const int one_row = min((int)threadIdx.x / D, rows_total - 1), one_col = (int)threadIdx.x % D;
  auto fold = [&](int q, const f32x4& acc, float m, float l) LS_INLINED {  // fold_split on these four columns
    if (!(l > 0.f)) return;
    const float m_new = fmaxf(run_m[q], m);
    const float a = softmax_exp<T>(run_m[q] - m_new);
    const float b = softmax_exp<T>(m - m_new);
#pragma unroll
    for (int e = 0; e < 4; ++e) run_acc[q][e] = run_acc[q][e] * a + acc[e] * b;
    run_l[q] = run_l[q] * a + l * b;
    run_m[q] = m_new;
  };

  if (LS_MUTANT_DEVICE(kMutantReversedFold)) {
    for (int s = n_splits - 1; s >= 0; --s) {
#pragma unroll
      for (int q = 0; q < MAXQ; ++q) {
        if (q * 256 + (int)threadIdx.x >= owned) continue;
        const long pr = pr_base + (long)row_of[q] * n_splits + s;
        fold(q, *reinterpret_cast<const f32x4*>(part_acc + pr * D + quad_of[q] * 4), part_ml[pr * 2], part_ml[pr * 2 + 1]);
      }
    }
  } else {
    // splits a batch: what fits the buffer, at most 32
    const int row_floats_max = STAGE / rows_total - ROW_PAD;
    const int batch = max(1, min(32, row_floats_max / D));
    const int row_stride = batch * D + ROW_PAD;      // floats
    const int per_row = batch * QUADS;               // 16-byte pieces of a row's batch
    const int total = rows_total * per_row;          // <= STAGE / 4
    f32x4 moved[PIECES];
    float2 moved_ml[2] = {float2{0.f, 0.f}, float2{0.f, 0.f}};  // up to 16 rows x 32 splits over 256 threads
    auto request = [&](int s0) LS_INLINED {  // the loads of the batch that starts at split s0, into registers
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const int idx = i * 256 + (int)threadIdx.x;
        const int row = min(idx / per_row, rows_total - 1);
        const int rest = idx - (idx / per_row) * per_row;
        const int u = rest / QUADS;
        const int piece = rest - u * QUADS;
        const long pr = pr_base + (long)row * n_splits + min(s0 + u, n_splits - 1);  // clamped: loaded, not used
        moved[i] = *reinterpret_cast<const f32x4*>(part_acc + pr * D + piece * 4);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int e = i * 256 + (int)threadIdx.x;
        if (e < rows_total * batch) {
          const int row = e / batch;
          const int u = e - row * batch;
          const long pr = pr_base + (long)row * n_splits + min(s0 + u, n_splits - 1);
          moved_ml[i] = *reinterpret_cast<const float2*>(part_ml + pr * 2);
        }
      }
    };
    auto put = [&](int buf) LS_INLINED {  // ... and from the registers to their place in LDS
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const int idx = i * 256 + (int)threadIdx.x;
        if (idx >= total) continue;
        const int row = idx / per_row;
        const int rest = idx - row * per_row;
        *reinterpret_cast<f32x4*>(&stage_acc[buf][row * row_stride + rest * 4]) = moved[i];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int e = i * 256 + (int)threadIdx.x;
        if (e < rows_total * batch) {
          stage_ml[buf][2 * e] = moved_ml[i].x;
          stage_ml[buf][2 * e + 1] = moved_ml[i].y;
        }
      }
    };
    request(0);
    int buf = 0;
    for (int s0 = 0; s0 < n_splits; s0 += batch, buf ^= 1) {
      put(buf);
      __syncthreads();  // the batch is in its buffer; the other buffer has been folded by every wave
      if (s0 + batch < n_splits) request(s0 + batch);
      const int count = min(batch, n_splits - s0);
      if (narrow) {
        // so few rows that every thread can have one column of one row: a quarter of the multiplications in
        // each thread's chain, and no wave stands by (the same operations on every element: the same bits)
        if ((int)threadIdx.x < rows_total * D) {
          const float* mine = &stage_acc[buf][one_row * row_stride + one_col];
          const float* ml = &stage_ml[buf][2 * one_row * batch];
          for (int u0 = 0; u0 < count; u0 += 4) {
            float acc4[4], m4[4], l4[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int u = min(u0 + k, count - 1);
              acc4[k] = mine[u * D];
              m4[k] = ml[2 * u];
              l4[k] = u0 + k < count ? ml[2 * u + 1] : 0.f;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const bool take = l4[k] > 0.f;
              const float m_new = fmaxf(run_m[0], m4[k]);
              const float a = softmax_exp<T>(run_m[0] - m_new);
              const float b = softmax_exp<T>(m4[k] - m_new);
              const float folded = run_acc[0][0] * a + acc4[k] * b;
              const float l_new = run_l[0] * a + l4[k] * b;
              run_acc[0][0] = take ? folded : run_acc[0][0];
              run_l[0] = take ? l_new : run_l[0];
              run_m[0] = take ? m_new : run_m[0];
            }
          }
        }
        continue;
      }
#pragma unroll
      for (int q = 0; q < MAXQ; ++q) {
        if (q * 256 + (int)threadIdx.x >= owned) continue;
        const float* mine = &stage_acc[buf][row_of[q] * row_stride + quad_of[q] * 4];
        const float* ml = &stage_ml[buf][2 * row_of[q] * batch];
        // Four splits' sums are read before the first of them is folded (the reads of one split take as long
        // as its fold), and a split of no weight is passed over by selects, not by a branch, so that nothing
        // stands between the reads and the chain of folds: fold_split's operations, the same bits.
        for (int u0 = 0; u0 < count; u0 += 4) {
          f32x4 acc4[4];
          float m4[4], l4[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int u = min(u0 + k, count - 1);
            acc4[k] = *reinterpret_cast<const f32x4*>(mine + u * D);
            m4[k] = ml[2 * u];
            l4[k] = u0 + k < count ? ml[2 * u + 1] : 0.f;
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const bool take = l4[k] > 0.f;
            const float m_new = fmaxf(run_m[q], m4[k]);
            const float a = softmax_exp<T>(run_m[q] - m_new);
            const float b = softmax_exp<T>(m4[k] - m_new);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float folded = run_acc[q][e] * a + acc4[k][e] * b;
              run_acc[q][e] = take ? folded : run_acc[q][e];
            }
            const float l_new = run_l[q] * a + l4[k] * b;
            run_l[q] = take ? l_new : run_l[q];
            run_m[q] = take ? m_new : run_m[q];
          }
        }
      }
    }
  }
  if (narrow) {
    if ((int)threadIdx.x < rows_total * D) {
      const float o = run_l[0] > 0.f ? run_acc[0][0] / run_l[0] : 0.f;
      out[(long)(item.q_off + one_row / G) * ldo + (long)(kvh * G + one_row % G) * D + one_col] = from_f32<T>(o);
    }
    return;
  }
#pragma unroll
  for (int q = 0; q < MAXQ; ++q) {
    if (q * 256 + (int)threadIdx.x >= owned) continue;
    const int r = row_of[q];
    T* p = out + (long)(item.q_off + r / G) * ldo + (long)(kvh * G + r % G) * D + quad_of[q] * 4;
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = run_l[q] > 0.f ? run_acc[q][e] / run_l[q] : 0.f;
    if (sizeof(T) == 2) {
      bf16x4 v;
      v[0] = (bf16_t)o[0]; v[1] = (bf16_t)o[1]; v[2] = (bf16_t)o[2]; v[3] = (bf16_t)o[3];
      *reinterpret_cast<bf16x4*>(p) = v;
    } else {
      *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
    }
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API
LS_DEFINE_MUTANT_API

using namespace ls;

extern "C" int ls_attn_head_dim() { return D; }
extern "C" int ls_attn_tile_keys() { return kTileKeys; }
extern "C" int ls_attn_split_keys() { return kSplitKeys; }
// Whether the staged kernel can have `bytes` of LDS: up to 64 KB always; above
// that the function attribute is raised once per kernel (the device offers
// 160 KB per workgroup); if that is refused the direct kernel runs instead.
static bool staged_fits(int dtype, size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  if (bytes > 160 * 1024) return false;
  static int state[2] = {0, 0};  // 0 unknown, 1 granted, -1 refused
  int& st = state[dtype == kF32 ? 0 : 1];
  if (st == 0) {
    hipError_t e = dtype == kF32
        ? hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_staged_kernel<float, false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes)
        : hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_staged_kernel<bf16_t, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) (void)hipGetLastError();
    st = e == hipSuccess ? 1 : -1;
  }
  return st == 1;
}

constexpr size_t kCoopExtra = 64 * 4 + NB * 64 * 4 + NB * 64 * 16;  // row maxima, block sums, probabilities
constexpr size_t kLdsLimit = 160 * 1024;

// The cooperative kernel: one or two buffers of a K and a V tile,
// two rows of page ids and the exchange buffers of the cooperative kernel.
constexpr size_t kCoopLdsExtra = kPageWindow * 16 * sizeof(int) + kCoopExtra + 2 * D * 4;  // + new key and value (FUSE)
constexpr int coop_bufs(size_t elem) {
  return 2 * (2 * kTileKeys * D * elem) + kCoopLdsExtra <= kLdsLimit ? 2 : 1;
}
template <typename T, int NBUF>
constexpr size_t coop_kernel_lds() { return NBUF * (2 * (size_t)kTileKeys * D * sizeof(T)) + kCoopLdsExtra; }

// Whether this instantiation can be launched (its LDS fits; above 64 KB the
// function attribute is raised once).
template <typename T, int NBUF, bool FUSE, bool SPANS = false>
static bool coop_kernel_ready() {
  constexpr size_t bytes = coop_kernel_lds<T, NBUF>();
  if (bytes > kLdsLimit) return false;
  if (bytes <= 64 * 1024) return true;
  static int state = 0;  // 0 unknown, 1 granted, -1 refused
  if (state == 0) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_coop_kernel<T, NBUF, FUSE, SPANS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) (void)hipGetLastError();
    state = e == hipSuccess ? 1 : -1;
  }
  return state == 1;
}

// Launch with two buffers (the next tile in flight while one is worked on)
// where they fit; when the grid brings at least two workgroups per CU, with
// one buffer instead, so that two workgroups share a CU and overlap each
// other's loads.
#ifndef LS_COOP_CROWDED_FROM
#define LS_COOP_CROWDED_FROM 512  // from this many workgroups on: one tile buffer each, two workgroups a CU
#endif
template <typename T, bool FUSE, bool SPANS>
static int launch_coop_as(dim3 grid, hipStream_t s, const void* q, long ldq, const void* k_pages, const void* v_pages,
                          int nkv, int page_size, int page_shift, const int* table, int table_stride, const void* seqs,
                          const void* items, void* out, long ldo, float* part_acc, float* part_ml, int G, float scale,
                          int window, DecodeFuse<T> fz, bool single_tile) {
  constexpr int BUFS = coop_bufs(sizeof(T));
  // one tile buffer (two workgroups a CU) where a second one could not be used: many workgroups, or items of
  // one tile each, which have no next tile to request ahead
  // (more workgroups than CUs but fewer than two a CU would be two rounds of one a CU with two buffers; with one
  // buffer they all run together: 48 requests of 8 kv heads 2.37 -> see the measurements in the planner)
  const bool crowded = (long)grid.x * grid.y >= LS_COOP_CROWDED_FROM || (long)grid.x * grid.y > compute_units() || single_tile;
#define LS_COOP(NBUF_)                                                                                              \
  hipLaunchKernelGGL((attention_coop_kernel<T, NBUF_, FUSE, SPANS>), grid, dim3(256), (coop_kernel_lds<T, NBUF_>()), s, \
                     (const AttnItem*)items, (const T*)q, ldq, fz.q_weight, fz.k_weight, fz.cos_table, fz.sin_table, G, \
                     nkv, (const T*)k_pages, (const T*)v_pages, page_size, page_shift, table, table_stride,            \
                     (const SeqMeta*)seqs, (T*)out, ldo, part_acc, part_ml, scale, window, fz)
  if (BUFS == 2 && !(crowded && coop_kernel_ready<T, 1, FUSE, SPANS>())) {
    if (!coop_kernel_ready<T, 2, FUSE, SPANS>()) return fail("attention: the cooperative kernel does not fit into LDS");
    LS_COOP(2);
  } else {
    if (!coop_kernel_ready<T, 1, FUSE, SPANS>()) return fail("attention: the cooperative kernel does not fit into LDS");
    LS_COOP(1);
  }
#undef LS_COOP
  return 0;
}

// ``spans``: items may hold several splits and leave a partial result for each (an instance of its own, so
// that the usual one-split items keep their code).
template <typename T, bool FUSE>
static int launch_coop(int spans, dim3 grid, hipStream_t s, const void* q, long ldq, const void* k_pages,
                       const void* v_pages, int nkv, int page_size, int page_shift, const int* table, int table_stride,
                       const void* seqs, const void* items, void* out, long ldo, float* part_acc, float* part_ml, int G,
                       float scale, int window, DecodeFuse<T> fz) {
  // spans: bit 0, items that leave partial results may hold several splits; bit 1, every item holds one tile
  const bool single_tile = (spans & 2) != 0;
  if (spans & 1)
    return launch_coop_as<T, FUSE, true>(grid, s, q, ldq, k_pages, v_pages, nkv, page_size, page_shift, table,
                                         table_stride, seqs, items, out, ldo, part_acc, part_ml, G, scale, window, fz,
                                         false);
  return launch_coop_as<T, FUSE, false>(grid, s, q, ldq, k_pages, v_pages, nkv, page_size, page_shift, table,
                                        table_stride, seqs, items, out, ldo, part_acc, part_ml, G, scale, window, fz,
                                        single_tile);
}

static bool coop_supported(int dtype) {
  return dtype == kF32 ? coop_kernel_ready<float, coop_bufs(4), false>()
                       : coop_kernel_ready<bf16_t, coop_bufs(2), false>();
}
// 1 if the cooperative kernel (variant 3, work items of at most 16 rows) can run for this dtype.
extern "C" int ls_attn_coop_supported(int dtype) { return coop_supported(dtype) ? 1 : 0; }

// The fused decode step (FUSE) stages the rotated query heads in the exchange
// buffers before the loop needs them: 16 rows of D elements.
static bool decode_fused_supported(int dtype) {
  const size_t elem = dtype == kF32 ? 4 : 2;
  if (16 * D * elem > (size_t)NB * 64 * 16) return false;
  return dtype == kF32 ? coop_kernel_ready<float, coop_bufs(4), true>()
                       : coop_kernel_ready<bf16_t, coop_bufs(2), true>();
}
// 1 if ls_attention_decode can run for this dtype.
extern "C" int ls_attn_decode_fused_supported(int dtype) { return decode_fused_supported(dtype) ? 1 : 0; }

// A step of single decoded tokens, with the per-head norm, the rotation and
// the cache write of qk_rope_kv fused in.  qkv [tokens, ld]: the raw fused
// projection (nq query heads, then nkv key heads, then nkv value heads); every
// request of `seqs` that the items name brings exactly one token.  The items
// are those of the cooperative variants.  cos/sin [table_positions][rot/2];
// max_pos is the largest position of the step.
extern "C" int ls_attention_decode(int dtype, const void* qkv, long ld, void* k_pages, void* v_pages, int nq, int nkv,
                                   int page_size, const int* table, int table_stride, const void* seqs,
                                   const void* items, int n_items, void* out, long ldo, float* part_acc,
                                   float* part_ml, float scale, int window, const float* q_weight,
                                   const float* k_weight, float eps, const float* cos_table, const float* sin_table,
                                   int rot, int table_positions, int max_pos, int write_kv, int spans, void* stream) {
  LS_REQUIRE(n_items > 0 && nkv > 0 && nq > 0 && nq % nkv == 0, "decode attention: bad sizes");
  const int G = nq / nkv;
  LS_REQUIRE(G <= 16, "decode attention: %d query heads per kv head, at most 16 fit a work item", G);
  LS_REQUIRE(page_size >= 8 && kTileKeys % page_size == 0 && (page_size & (page_size - 1)) == 0,
             "decode attention: page size %d must be a power of two from 8 that divides the key tile %d", page_size,
             kTileKeys);
  LS_REQUIRE(ld % 8 == 0 && ldo % 4 == 0 && ld >= (long)(nq + 2 * nkv) * D && ldo >= (long)nq * D,
             "decode attention: row strides ld=%ld ldo=%ld do not fit the heads", ld, ldo);
  LS_REQUIRE(reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 && reinterpret_cast<uintptr_t>(v_pages) % 16 == 0,
             "decode attention: operands must be 16-byte aligned");
  LS_REQUIRE(rot >= 0 && head16_supported(D, rot), "decode attention: rotary_dim %d must be even and at most %d",
             rot, D);
  LS_REQUIRE((!q_weight || reinterpret_cast<uintptr_t>(q_weight) % 16 == 0) &&
                 (!k_weight || reinterpret_cast<uintptr_t>(k_weight) % 16 == 0) &&
                 (!cos_table || (reinterpret_cast<uintptr_t>(cos_table) % 16 == 0 &&
                                 reinterpret_cast<uintptr_t>(sin_table) % 16 == 0)),
             "decode attention: norm weights and rotation tables must be 16-byte aligned");
  LS_REQUIRE(!cos_table || (sin_table && table_positions > max_pos),
             "decode attention: rotation tables hold %d positions, the step reaches %d", table_positions, max_pos);
  LS_REQUIRE(decode_fused_supported(dtype), "decode attention: the fused kernel does not fit into LDS for this head size");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid(n_items, nkv);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  int rc = 0;
  if (dtype == kF32) {
    DecodeFuse<float> fz{q_weight, k_weight, eps, cos_table, sin_table, rot, nq, write_kv, (float*)k_pages, (float*)v_pages};
    rc = launch_coop<float, true>(spans, grid, s, qkv, ld, k_pages, v_pages, nkv, page_size, page_shift, table, table_stride,
                                  seqs, items, out, ldo, part_acc, part_ml, G, scale, window, fz);
  } else if (dtype == kBF16) {
    DecodeFuse<bf16_t> fz{q_weight, k_weight, eps, cos_table, sin_table, rot, nq, write_kv, (bf16_t*)k_pages,
                          (bf16_t*)v_pages};
    rc = launch_coop<bf16_t, true>(spans, grid, s, qkv, ld, k_pages, v_pages, nkv, page_size, page_shift, table, table_stride,
                                   seqs, items, out, ldo, part_acc, part_ml, G, scale, window, fz);
  } else {
    return fail("decode attention: unknown dtype %d", dtype);
  }
  if (rc != 0) return rc;
  return check_launch("attention (decode, fused)");
}

// The wide kernel: two buffers of a K and a V tile, and two rows of page ids.  Eight waves (row blocks of
// 128) or, for steps with so few rows that 128-row blocks would leave CUs without work, four (blocks of 64).
constexpr int kWideWaves = 8;
constexpr int kNarrowWaves = 4;
static size_t wide_lds_bytes(int dtype) { return 4 * (size_t)kTileKeys * D * (dtype == kF32 ? 4 : 2) + kPageWindow * 16 * sizeof(int); }
template <typename T, int NW>
static bool wide_kernel_ready(size_t bytes) {
  static int state = 0;  // 0 unknown, 1 granted, -1 refused
  if (state == 0) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_wide_kernel<T, NW>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) (void)hipGetLastError();
    state = e == hipSuccess ? 1 : -1;
  }
  return state == 1;
}
static bool wide_supported(int dtype) {
  const size_t bytes = wide_lds_bytes(dtype);
  if (bytes > kLdsLimit) return false;
  if (bytes <= 64 * 1024) return true;
  return dtype == kF32 ? (wide_kernel_ready<float, kWideWaves>(bytes) && wide_kernel_ready<float, kNarrowWaves>(bytes))
                       : (wide_kernel_ready<bf16_t, kWideWaves>(bytes) && wide_kernel_ready<bf16_t, kNarrowWaves>(bytes));
}
// 1 if the wide kernel (variants 4 and 5) can run for this dtype.
extern "C" int ls_attn_wide_supported(int dtype) { return wide_supported(dtype) ? 1 : 0; }
// Rows of one work item's row block: AttnItem.row_block counts blocks of this many rows.
extern "C" int ls_attn_block_rows(int variant) {
  return variant == 4 ? 16 * kWideWaves : variant == 5 ? 16 * kNarrowWaves : 64;
}

// variant: 4 and 5 run the wide kernel (row blocks of ls_attn_block_rows(variant) rows: 128 and 64);
// variant: 3 runs the cooperative kernel (all items must have at most 16 rows);
// variant: 0 picks the staged kernel where its tiles fit into LDS and the
// direct one elsewhere, 1 forces the direct kernel, 2 the staged one.
// q [tokens, ldq]: head h of a token at columns [h*D, (h+1)*D).  out likewise
// with ldo.  k_pages [pages][nkv][page_size][D], v_pages [pages][nkv][D][page_size].
// table [rows][table_stride] int32 (page id or -1).  items: n_items AttnItem (16 ints each).
extern "C" int ls_attention(int dtype, const void* q, long ldq, const void* k_pages, const void* v_pages, int nkv,
                            int page_size, const int* table, int table_stride, const void* seqs, const void* items,
                            int n_items, void* out, long ldo, float* part_acc, float* part_ml, int G, float scale,
                            int window, int variant, int max_rows, int spans, void* stream) {
  LS_REQUIRE(n_items > 0 && nkv > 0 && G > 0, "attention: bad sizes (items %d, kv heads %d, group %d)", n_items, nkv, G);
  LS_REQUIRE(page_size >= 4 && page_size % 4 == 0 && kTileKeys % page_size == 0,
             "attention: page size %d must be a multiple of 4 that divides the key tile %d", page_size, kTileKeys);
  LS_REQUIRE(ldq % 8 == 0 && ldo % 4 == 0, "attention: row strides ldq=%ld ldo=%ld are not vector aligned", ldq, ldo);
  LS_REQUIRE(ldq >= (long)nkv * G * D && ldo >= (long)nkv * G * D, "attention: row strides shorter than the heads");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 && reinterpret_cast<uintptr_t>(v_pages) % 16 == 0,
             "attention: operands must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid(n_items, nkv);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  LS_REQUIRE((1 << page_shift) == page_size, "attention: page size %d is not a power of two", page_size);
  const size_t elem = dtype == kF32 ? 4 : 2;
  const size_t lds_bytes = 2 * (size_t)kTileKeys * D * elem;
  if (variant == 3) {
    LS_REQUIRE(max_rows <= 16, "attention: the cooperative variants take work items of at most 16 rows, got %d",
               max_rows);
    LS_REQUIRE(coop_supported(dtype), "attention: the cooperative variant does not fit into LDS for this head size");
    LS_REQUIRE(page_size >= 8, "attention: the cooperative variant needs pages of at least 8 keys, got %d", page_size);
    int rc = 0;
    if (dtype == kF32)
      rc = launch_coop<float, false>(spans, grid, s, q, ldq, k_pages, v_pages, nkv, page_size, page_shift, table, table_stride,
                                     seqs, items, out, ldo, part_acc, part_ml, G, scale, window, DecodeFuse<float>{});
    else if (dtype == kBF16)
      rc = launch_coop<bf16_t, false>(spans, grid, s, q, ldq, k_pages, v_pages, nkv, page_size, page_shift, table,
                                      table_stride, seqs, items, out, ldo, part_acc, part_ml, G, scale, window,
                                      DecodeFuse<bf16_t>{});
    else
      return fail("attention: unknown dtype %d", dtype);
    if (rc != 0) return rc;
    return check_launch("attention (cooperative)");
  }
  if (variant == 4 || variant == 5) {
    LS_REQUIRE(wide_supported(dtype), "attention: the wide variant does not fit into LDS for this head size");
    LS_REQUIRE(page_size >= 8, "attention: the wide variant needs pages of at least 8 keys, got %d", page_size);
    LS_REQUIRE(dtype == kF32 || dtype == kBF16, "attention: unknown dtype %d", dtype);
    const size_t bytes = wide_lds_bytes(dtype);
#define LS_WIDE(T_, NW_)                                                                                          \
  hipLaunchKernelGGL((attention_wide_kernel<T_, NW_>), grid, dim3(64 * NW_), bytes, s, (const T_*)q, ldq,          \
                     (const T_*)k_pages, (const T_*)v_pages, nkv, page_size, page_shift, table, table_stride,       \
                     (const SeqMeta*)seqs, (const AttnItem*)items, (T_*)out, ldo, part_acc, part_ml, G, scale, window)
    if (dtype == kF32) {
      if (variant == 4) LS_WIDE(float, kWideWaves); else LS_WIDE(float, kNarrowWaves);
    } else {
      if (variant == 4) LS_WIDE(bf16_t, kWideWaves); else LS_WIDE(bf16_t, kNarrowWaves);
    }
#undef LS_WIDE
    return check_launch("attention (wide)");
  }
  const bool staged = variant != 1 && staged_fits(dtype, lds_bytes);
  LS_REQUIRE(variant != 2 || staged, "attention: the staged variant needs %zu bytes of LDS, which is not available",
             lds_bytes);
  if (dtype == kF32) {
    if (staged)
      hipLaunchKernelGGL((attention_staged_kernel<float, false>), grid, dim3(256), lds_bytes, s, (const float*)q,
                         ldq, (const float*)k_pages, (const float*)v_pages, nkv, page_size, page_shift, table,
                         table_stride, (const SeqMeta*)seqs, (const AttnItem*)items, (float*)out, ldo, part_acc,
                         part_ml, G, scale, window);
    else
      hipLaunchKernelGGL(attention_direct_kernel<float>, grid, dim3(256), 0, s, (const float*)q, ldq,
                         (const float*)k_pages, (const float*)v_pages, nkv, page_size, table, table_stride,
                         (const SeqMeta*)seqs, (const AttnItem*)items, (float*)out, ldo, part_acc, part_ml, G, scale,
                         window);
  } else if (dtype == kBF16) {
    if (staged)
      hipLaunchKernelGGL((attention_staged_kernel<bf16_t, true>), grid, dim3(256), lds_bytes, s, (const bf16_t*)q,
                         ldq, (const bf16_t*)k_pages, (const bf16_t*)v_pages, nkv, page_size, page_shift, table,
                         table_stride, (const SeqMeta*)seqs, (const AttnItem*)items, (bf16_t*)out, ldo, part_acc,
                         part_ml, G, scale, window);
    else
      hipLaunchKernelGGL(attention_direct_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)q, ldq,
                         (const bf16_t*)k_pages, (const bf16_t*)v_pages, nkv, page_size, table, table_stride,
                         (const SeqMeta*)seqs, (const AttnItem*)items, (bf16_t*)out, ldo, part_acc, part_ml, G, scale,
                         window);
  } else {
    return fail("attention: unknown dtype %d", dtype);
  }
  return check_launch("attention");
}

extern "C" int ls_attention_combine(int dtype, const void* seqs, const void* items, int n_items, int nkv,
                                    const float* part_acc, const float* part_ml, void* out, long ldo, int G,
                                    int max_rows, void* stream) {
  // max_rows: the most rows (tokens times query heads a kv head) any item's request brings, or 0 if unknown;
  // up to 16 rows the kernel that shares a row's columns among the waves is taken.
  LS_REQUIRE(n_items > 0 && nkv > 0 && G > 0 && max_rows >= 0, "combine: bad sizes");
  LS_REQUIRE(ldo % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0, "combine: output not vector aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid(n_items, nkv);
  const bool few = max_rows > 0 && max_rows <= 16;
#define LS_COMBINE(KERNEL_, T_)                                                                              \
  hipLaunchKernelGGL(KERNEL_<T_>, grid, dim3(256), 0, s, (const SeqMeta*)seqs, (const CombineItem*)items, \
                     part_acc, part_ml, (T_*)out, ldo, G)
  if (dtype == kF32) {
    if (few) LS_COMBINE(combine_few_rows_kernel, float); else LS_COMBINE(combine_kernel, float);
  } else if (dtype == kBF16) {
    if (few) LS_COMBINE(combine_few_rows_kernel, bf16_t); else LS_COMBINE(combine_kernel, bf16_t);
  } else {
    return fail("combine: unknown dtype %d", dtype);
  }
#undef LS_COMBINE
  return check_launch("combine");
}

// The entry points that a list of launches may name (see ls_run_list of the core library).
#define LS_ATTENTION_LISTED(X) X(ls_attention) X(ls_attention_decode) X(ls_attention_combine)
LS_DEFINE_LISTED_CALLS(LS_ATTENTION_LISTED)
