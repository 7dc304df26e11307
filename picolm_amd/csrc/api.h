// C entry points of libpicolm_hip.so.  Pointers are device pointers unless said otherwise;
// every function returns 0 on success and a negative code with a message in
// picolm_last_error() otherwise.  Nothing here synchronises: work is queued on `stream`.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// element types of tensors and buffers: float, or bfloat16 stored as 16 bits
#ifndef PICOLM_ELEMENT_TYPES
#define PICOLM_ELEMENT_TYPES
enum { PICOLM_F32 = 0, PICOLM_BF16 = 1 };
#endif

const char* picolm_last_error(void);
// leaves a message for picolm_last_error(): for code outside the library that fails a call of the
// library's (an operation of the caller's inside an engine's program)
void picolm_set_error_message(const char* message);
int picolm_abi_version(void);
int picolm_device_check(void);     // 0 if the current device is a gfx950

// Sweeps `src` once, each workgroup a contiguous share in whole rounds of 32 KB (picolm_read_probe_bytes
// says how many bytes that reads), with non-temporal loads if `streaming`; for bandwidth measurements.
int picolm_read_probe(const void* src, size_t bytes, void* sink, int blocks, int streaming, hipStream_t stream);
size_t picolm_read_probe_bytes(size_t bytes, int blocks);

// runs blocks*4 waves of `iters` x 8 MFMAs (32x32x16 bf16) on registers, on small integers or
// (random_operands != 0) on pseudo-random values of the size of real data, which the GPU's power
// limit slows down; for MFMA-rate measurements
int picolm_mfma_probe(void* sink, int blocks, int iters, int random_operands, hipStream_t stream);

int picolm_embed(const void* table, int table_dt, const int32_t* tokens, float* x, int T, int D,
                 int V, hipStream_t stream);
int picolm_gather_i32(int32_t* out, const int32_t* src, const int32_t* index, int n, hipStream_t stream);   // out[i] = src[index[i]]
int picolm_rmsnorm(const float* x, const float* w, void* out, int out_dt, const int32_t* rows,
                   int n_rows, int D, float eps, hipStream_t stream);
int picolm_rope_kv_store(const float* qkv, void* q_out, void* k_pages, void* v_pages, int dt,
                         const float* cos_t, const float* sin_t, int style, const int32_t* tok_pos,
                         const int32_t* tok_page /* physical cache page of every token */, int T, int H, int G,
                         int d, const int32_t* rows /* null: rows 0..T-1 */, hipStream_t stream);

// Keys (rotated) and values of a prefill step into the cache, over the attention kernel's tiles
// (tile t: up to tile_tokens new tokens of sequence tile_seq[t] from its tile_q0[t]-th on); q is
// left alone.  d in multiples of 4.
int picolm_kv_store_tiles(const float* qkv, void* k_pages, void* v_pages, int dt, const float* cos_t,
                          const float* sin_t, int style, const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                          int tile_tokens, const int32_t* seq_slot, const int32_t* seq_pos0, const int32_t* seq_nnew,
                          const int32_t* cu_seqlens, const int32_t* page_table, int max_pages, int ring_pages, int H,
                          int G, int d, hipStream_t stream);

int picolm_gemm_generic(const void* A, int a_dt, const void* W, int w_dt, void* C, int c_dt, int M,
                        int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue,
                        hipStream_t stream);

// bf16 operands on the matrix cores; K and the row strides must be multiples of 8.
int picolm_gemm_skinny(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                       int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream);
int picolm_gemm_tiled(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                      int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream);

// ws: splits * M * N floats; variants 9 and up
int picolm_gemm_tiled_splitk(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                             int64_t ldw, int64_t ldc, int epilogue, int variant, int splits, float* ws,
                             hipStream_t stream);

// A decode step's products with an RMSNorm split between them.  A product with the accumulating
// epilogue can prepare the norm that follows: next_h[M][ldc] = bf16(x * next_w) and
// next_ssq[next_parts][rows], one row of partial sums of x^2 per workgroup.  A product whose input
// rows are such a next_h takes ssq[n_parts][rows], the norm's row length and eps and multiplies
// its sums by 1 / sqrt(sum / len + eps).  Up to 16 rows (rows = 16): skinny variant 0/1 (either
// role), 7, or tiled != 0 with tile variant 12/13 (taking only).  17 to 64 rows (rows = 64): tiled,
// variant 12 (13 up to 32 rows); cut along K (splits > 1, ws of splits * M * N floats, N a multiple of 1024) either
// role, uncut taking only.
// More than 64 rows (rows = a multiple of 64 of at least M, sums for every row): the tiled product
// by shape, either role, cut along K when ws (ws_floats floats) is given and the shape has tiles for
// half of the CUs or fewer; picolm_gemm_tiled_norm_parts gives the shares it leaves (0: it cannot).
int picolm_gemm_tiled_norm_parts(int M, int N, int K, int64_t ws_floats);
int picolm_gemm_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                       int64_t ldw, int64_t ldc, int epilogue, int tiled, int variant, int splits, float* ws,
                       int64_t ws_floats, const float* next_w, void* next_h, float* next_ssq, int next_parts, const float* ssq,
                       int n_parts, int norm_len, float eps, int rows, hipStream_t stream);

// The product a layer asks for: picks the kernel for the operands' types and sizes (linear.hip).
// Row-major contiguous A[M][K], W[N][K], C[M][N] (N/2 with the gated epilogue 2).  next_*: with
// the accumulating epilogue 1, also prepare the RMSNorm that follows (next_h[M][N] bf16, next_ssq
// [next_parts][rows] with rows = picolm_linear_norm_rows(M), next_parts =
// picolm_linear_norm_parts(M, N, K)); ssq, n_parts, norm_len, eps: A is such a next_h.  Either
// role needs picolm_linear_links_norms to say yes.  ws: picolm_linear_workspace_floats() floats for
// products cut along K, or null.
int64_t picolm_linear_workspace_floats(void);
int picolm_linear_norm_rows(int M);
int picolm_linear_medium_splits(int M, int N, int K);    // parts along K of a product of 17..64 rows
int picolm_linear_norm_parts(int M, int N, int K);
int picolm_linear_links_norms(const void* a, int a_dt, const void* w, int w_dt, int c_dt, int M, int N, int K,
                              int epilogue, int prepares);
int picolm_linear(const void* A, int a_dt, const void* W, int w_dt, void* C, int c_dt, int M, int N, int K, int epilogue,
                  const float* next_w, void* next_h, float* next_ssq, int next_parts, const float* ssq, int n_parts,
                  int norm_len, float eps, float* ws, hipStream_t stream);

// Within a group's part of a page, K[64][d] and V^T[d][64] lie as plain arrays, except in bfloat16
// pages of a head size that is a multiple of 32 up to 256: those are in the order of the matrix-core
// kernels' operands.
// Fills k_idx[key * d + i] and v_idx[i * 64 + key] with the offsets of K[key][i] and V^T[i][key].
int picolm_kv_page_order(int dt, int d, int32_t* k_idx, int32_t* v_idx);
int picolm_attn_prefill_tile_rows(void);
int picolm_attn_prefill_generic(const void* q, const void* k_pages, const void* v_pages, void* out,
                                int dt, const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                                const int32_t* seq_slot, const int32_t* seq_pos0,
                                const int32_t* seq_nnew, const int32_t* cu_seqlens,
                                const int32_t* page_table, int max_pages, int ring_pages, int H,
                                int G, int d, int window, float scale, hipStream_t stream);
// Decode (row i of q and out is sequence i).  chunk_list is the step's work list of 1 + n_chunks
// entries of eight ints: a header whose first int says how many entries are in use, then
// {sequence, which chunk of the sequence, position of the new token, cache slot, physical pages of
// the chunk's first four pages}; workgroup x of the launch takes entry 1 + x.  A chunk is
// pages_per_chunk pages; a sequence has at most max_splits chunks, and where it has several their
// partial results (partial: [n_seq][H][max_splits][d+2] floats) are combined by a merge kernel
// that follows.
int picolm_attn_decode_generic(const void* q, const void* k_pages, const void* v_pages, void* out,
                               float* partial, int dt, int n_seq, const int32_t* chunk_list, int n_chunks,
                               int pages_per_chunk, int max_splits, const int32_t* seq_pos0,
                               const int32_t* page_table, int max_pages, int ring_pages, int H, int G, int d,
                               int window, float scale, hipStream_t stream);

// bf16 attention on the matrix cores: head sizes in multiples of 32 up to 256 (the cache's pages of
// such heads are in the order of the MFMA operands); picolm_attn_mfma_fits: and a group's query
// heads, of which a decode workgroup keeps partial results in LDS, fit there
int picolm_attn_mfma_takes(int d);
int picolm_attn_mfma_fits(int H, int G, int d);
int picolm_attn_prefill_mfma_heads(int H, int G);
int picolm_attn_prefill_mfma_tile_tokens(int H, int G);
int picolm_attn_prefill_mfma(const void* q, const void* k_pages, const void* v_pages, void* out,
                             const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                             const int32_t* seq_slot, const int32_t* seq_pos0, const int32_t* seq_nnew,
                             const int32_t* cu_seqlens, const int32_t* page_table, int max_pages,
                             int ring_pages, int H, int G, int d, int window, float scale, hipStream_t stream);
// The same with q taken from the float rows qkv[T][(H+2G)*d] and rotated inside the kernel (tables
// as in picolm_rope_kv_store, both null for no rotation); the step's keys and values must be in
// the cache already.
int picolm_attn_prefill_rotates_q(int T);      // whether a step of T tokens should take this way (long prompts gain, short ones lose)
int picolm_attn_prefill_rope_mfma(const float* qkv, const void* k_pages, const void* v_pages, void* out,
                                  const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                                  const int32_t* seq_slot, const int32_t* seq_pos0, const int32_t* seq_nnew,
                                  const int32_t* cu_seqlens, const int32_t* page_table, int max_pages,
                                  int ring_pages, int H, int G, int d, int window, float scale,
                                  const float* cos_t, const float* sin_t, int style, hipStream_t stream);
int picolm_attn_decode_mfma_waves(int n_seq, int H, int G);      // waves a decode workgroup will have
// chunks_done: n_seq * G * ceil(H/G / 32) counters that are zero when the call starts and zero again
// when its kernel has run: the workgroup that finishes a sequence's last chunk combines the chunks,
// and no merge kernel runs.  Null: the merge kernel combines them.
int picolm_attn_decode_mfma(const void* q, const void* k_pages, const void* v_pages, void* out, float* partial,
                            int n_seq, const int32_t* chunk_list, int n_chunks, int pages_per_chunk,
                            int max_splits, const int32_t* seq_pos0, const int32_t* page_table, int max_pages,
                            int ring_pages, int H, int G, int d, int window, float scale, int32_t* chunks_done,
                            hipStream_t stream);

// Rotation, cache write and attention of a decode step in one launch: q, k, v of the new tokens are
// the float rows qkv[n_seq][(H+2G)*d]; tok_page[i] is the physical page for sequence i's new key
// and value; cos_t, sin_t [positions][d/2], or both null for no rotation; style as in picolm_rope_kv_store.
int picolm_attn_decode_rope_mfma(const float* qkv, void* k_pages, void* v_pages, void* out, float* partial,
                                 int n_seq, const int32_t* chunk_list, int n_chunks, int pages_per_chunk,
                                 int max_splits, const int32_t* seq_pos0, const int32_t* page_table,
                                 int max_pages, int ring_pages, int H, int G, int d, int window, float scale,
                                 const float* cos_t, const float* sin_t, int style, const int32_t* tok_page,
                                 int32_t* chunks_done, hipStream_t stream);

int picolm_argmax_scratch_floats(int n_rows, int V);
int picolm_argmax(const float* logits, int32_t* out, int n_rows, int V, int64_t ld, float* scratch,
                  hipStream_t stream);
// picolm_argmax for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid it).  It has no counterpart in picolm.  The partial
// results go to an array of picolm_argmax_static_max_floats() floats (256 KiB) that the library
// keeps in each GPU's memory for the life of the process; 2 * n_rows * ceil(V / 4096) floats
// beyond that are refused with an error.  It allocates and frees nothing.  All calls on one GPU
// share that GPU's array: two calls that overlap there (different streams, or threads without an
// order between them) race; calls queued on one stream do not.
int picolm_argmax_static_max_floats(void);
int picolm_argmax_static(const float* logits, int32_t* out, int n_rows, int V, int64_t ld, hipStream_t stream);
// rng_states[state_index ? state_index[row] : row] is one xorshift64 state per sequence,
// advanced by one draw when temperature > 0.
// With a top_k small enough the row is cut into slices for many workgroups, which need scratch
// memory: picolm_sample_scratch_bytes says how much (0: this case is one workgroup per row and
// needs none); `scratch` may be null, then one workgroup per row does all the work.
int picolm_sample_scratch_bytes(int n_rows, int V, float temperature, int top_k);
int picolm_sample(const float* logits, int64_t ld, int n_rows, int V, float temperature, int top_k,
                  float top_p, float min_p, uint64_t* rng_states, const int32_t* state_index,
                  int32_t* out, void* scratch, int64_t scratch_bytes, hipStream_t stream);

#ifdef __cplusplus
}
#endif
