// The C interface of the core library (core.hip, gemm.hip).
//
// Conventions shared by every entry point: dtype is 0 for float32 and 1 for
// bfloat16; pointers are device pointers unless said otherwise; `stream` is a
// hipStream_t passed as void*; the return value is 0 or a negative code, and
// ls_last_error() then returns the message.  Shapes and alignment are checked
// on the host before a kernel is launched.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

const char* ls_last_error();

// Rows of the residual stream.
int ls_embed(int dtype, const int* tokens, const void* table, float* out, int n_tokens, int vocab, int width,
             long ld_out, void* stream);
int ls_rmsnorm(int dtype, const float* x, const float* weight, void* out, const int* rows, int n_rows, int width,
               long ldx, long ld_out, float eps, void* stream);
int ls_add_rmsnorm(int dtype, float* h, const float* P, int slices, int p_rows, const float* weight, void* out,
                   const int* rows, int n_rows, int width, long ldh, long ld_out, float eps, void* stream);
int ls_qk_rope_kv(int dtype, void* qkv, long ld, int n_tokens, int nq, int nkv, int d, const float* q_weight,
                  const float* k_weight, float eps, const float* cos_table, const float* sin_table, int rot,
                  int table_positions, const int* tok_seq, const int* tok_pos, const void* seqs, const int* table,
                  int table_stride, void* k_pages, void* v_pages, int page_size, int write_kv, void* stream);
int ls_swiglu(int dtype, const void* gu, void* out, int rows, int inter, long ld_in, long ld_out, void* stream);

// Bias and activation on float rows: out = act(x + bias), times (x[:, width:] + bias[width:]) when gated.
// out_dtype 0 float32, 1 bfloat16; act 0 none, 1 SiLU, 2 GELU (tanh), 3 GELU (erf), 4 ReLU.
int ls_bias_act(int out_dtype, const float* x, long ldx, const float* bias, void* out, long ldo, int rows, int width,
                int act, int gated, void* stream);

// Temperature / nucleus sampling of n rows.  requests: n records of 32 bytes on the device (int row of logits,
// float temperature > 0, double top_p, unsigned key0, key1 (halves of seed XOR k(uid)), unsigned position low, high:
// the draw is Philox-4x32-10 of them); token ids to out[i].  scratch: ls_sample_scratch_bytes(n, vocab) bytes of
// device memory, 256-byte aligned.  any_nucleus: 0 if every top_p is >= 1.  scatter: token ids go to out[row of the
// record] instead of out[i].
long ls_sample_scratch_bytes(int n, int vocab);
int ls_sample_top_p(const float* logits, long ld, const void* requests, int* out, void* scratch, long scratch_bytes,
                    int n, int vocab, int any_nucleus, int scatter, void* stream);

// Arg-max of float rows, lowest index among equal maxima.  Rows wider than one chunk leave the
// chunks' winners in `scratch` (2 * rows * ls_argmax_chunks(width) 4-byte words, device memory
// the caller brings) for a second small launch.
int ls_argmax_chunks(int width);
int ls_argmax(const float* x, int* out, int rows, int width, long ld, void* scratch, long scratch_words,
              void* stream);

// The same arg-max for callers that cannot allocate device memory and have no workspace to
// hand over: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  This entry point has no counterpart in the reference engine (whose sampler runs
// in a framework that allocates freely); it exists for those callers alone.  The chunks'
// winners go to an array that lives in the library's device image, LS_ARGMAX_STATIC_PAIRS
// (row, chunk) pairs large (128 KiB on every GPU the library runs on, held until the process
// ends); a call with rows * ls_argmax_chunks(width) beyond that is refused with an error, and
// nothing is launched.  No hipMalloc, hipFree or other allocating call is made.  Every (row,
// chunk) entry the second launch reads is written by the first, so nothing has to be cleared
// between calls; but all calls on one GPU share the array, so two calls that overlap in time
// on one GPU (different streams, or different threads) race: order them on one stream.  The
// address of the array on the current device is looked up once per device, at the first call
// there; make that call outside graph capture.  Same kernels and same bits as ls_argmax.
#define LS_ARGMAX_STATIC_PAIRS 16384
int ls_argmax_static(const float* x, int* out, int rows, int width, long ld, void* stream);

int ls_advance_decode(int* meta, long meta_ints, int n_seqs, int off_tokens, const int* picked, int* ring,
                      int* counter, int off_runs, int n_runs, void* stream);

// Matrix products C = X W^T with a fixed summation order (see gemm.hip).
int ls_gemm(int dtype, int epilogue, const void* X, const void* W, void* C, int M, int N, int K, long ldx, long ldc,
            const float* norm_w, float eps, int out_cols, void* stream);
int ls_gemm_kslice(int K);
int ls_gemm_slices_count(int K);
int ls_gemm_slices_max_rows(int dtype, int K);
int ls_gemm_slices(int dtype, const void* X, const void* W, float* P, int M, int N, int K, long ldx, void* stream);
int ls_gemm_slices_folded_ok(int dtype, int M, int N, int K, int head_dim, int splits);
int ls_gemm_slices_folded(int dtype, const float* part_acc, const float* part_ml, int splits, int head_dim,
                          const void* W, float* P, int M, int N, int K, void* stream);

// A list of launches in one call.  `words` holds records of 8-byte words one after the other:
//   [the address of a library's ls_call_listed, the entry point's ls_listed_index there, n, n argument words]
// (an integer, a pointer, or a float's bits in the low half of its word).  The calls are made in order on the
// calling thread; the first that fails ends the run: its code is returned, `failed_at` (if not null) gets the
// offset of its record, and the message is with the library that the record names.
int ls_listed_index(const char* name);
int ls_call_listed(int index, const long long* words, int n);
int ls_run_list(const long long* words, long n_words, long* failed_at);

#ifdef __cplusplus
}
#endif
