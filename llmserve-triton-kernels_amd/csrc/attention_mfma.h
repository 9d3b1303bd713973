// Entry points of attention_mfma.hip (the library libllms_attention_mfma_*.so).
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

// bfloat16 causal attention over the paged cache for the requests [seq_begin, seq_begin + n_seqs) of a step
// (see the comment at its definition).  With num_splits > 1 the caller brings the workspace for the partial
// results: ws_o [rows * heads * splits * head_dim] and ws_ml [rows * heads * splits * 2] floats; and, if it wants the
// shares of a decoding launch added up by the workgroup that finishes last rather than by a second kernel, n_arrive
// counters that are zero and stay zero (arrive; null: the second kernel).
int llms_attention_mfma(void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                        const int* cu_seqlens, const int* context_lens, int seq_begin, int n_seqs, int max_new,
                        int token_begin, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int block_size,
                        int window, float scale, int split_waves, int num_splits, int waves, float* ws_o,
                        float* ws_ml, unsigned* arrive, int n_arrive, hipStream_t stream);

// The split decode attention (every request brings one token; its keys are dealt to `waves` = 4 or 8 waves and
// to num_splits >= 2 workgroups, merged in fixed order) for callers that cannot allocate: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
// (whose attention is a library call that allocates as it pleases).  The arguments are those of
// llms_attention_mfma without the workspace: the partial results go through a fixed array in device memory
// that the library owns, LLMS_ATTN_SCRATCH_BYTES per GPU for the life of the process.  The call allocates and
// frees nothing (no hipMalloc, no hipFree, no allocating library routine); at its first call on a device it
// asks the runtime once for the array's address there (and the runtime, if nothing of this library has run on
// that device yet, loads the library's code there, array included): make the first call outside a capture.
//   cu_seqlens on the device must describe rows inside [token_begin, token_begin + n_tokens): the partial results
//   are indexed by those rows, and a column whose row lies beyond is left out.
//   Limit: (token_begin + n_tokens) * n_heads * num_splits * (head_dim + 2) * 4 bytes <= LLMS_ATTN_SCRATCH_BYTES,
//   e.g. 64 rows x 32 heads x 8 splits at head_dim 128; a larger launch is refused (return code 1, message
//   on stderr) and nothing runs.
//   All calls on one GPU share that GPU's array, which keeps what the last call left in it; nothing in it needs
//   clearing between calls.  Two calls that overlap in time on one GPU (different streams, or threads on
//   different streams) race on it: keep calls on one stream, or order them yourself.
#define LLMS_ATTN_SCRATCH_BYTES (8u << 20)
int llms_attention_decode_noalloc(void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                                  const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                                  const int* cu_seqlens, const int* context_lens, int seq_begin, int n_seqs,
                                  int token_begin, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                  int block_size, int window, float scale, int num_splits, int waves,
                                  hipStream_t stream);

}  // extern "C"
