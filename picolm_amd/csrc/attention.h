// Arguments shared by the attention kernels over the paged cache.
#pragma once
#include <stdint.h>

#define NEG_BIG (-1e30f)

struct AttnArgs {
    const void* q;            // [T][H*d]
    const void* k_pages;      // [n_pages][G][PAGE][d]
    const void* v_pages;      // [n_pages][G][d][PAGE]
    void* out;                // [T][H*d]
    float* partial;           // decode: [n_seq][H][max_splits][d+2]
    const int32_t* tile_seq;  // prefill: sequence of each tile
    const int32_t* tile_q0;   // prefill: first new-token index of each tile
    const int32_t* seq_slot;
    const int32_t* seq_pos0;  // tokens the sequence held before this step
    const int32_t* seq_nnew;
    const int32_t* cu_seqlens;  // first token row of each sequence in this step
    const int32_t* page_table;
    int max_pages, ring_pages;
    int H, G, d, window;
    float scale;
    int decode;     // 0 prefill tiles, 1 decode groups
    // decode: workgroup x is chunk x of the step's work list: pages_per_chunk pages of one sequence
    const int32_t* chunk_seq;   // sequence of each chunk, or -1 for an unused entry
    const int32_t* chunk_idx;   // which chunk of its sequence
    int pages_per_chunk;
    int max_splits;             // chunks a sequence can have: stride of `partial`
};

// What a decode workgroup has to do.  A sequence whose visible pages fit one chunk is finished by
// its workgroup; otherwise every chunk leaves (max, sum, acc) in `partial` and the merge kernel
// combines them.  The host's work list is built from the same arithmetic.
struct DecodeWork {
    int seq, split, page_lo, page_hi, n_chunks;
};
__device__ __forceinline__ int decode_first_page(const AttnArgs& a, int qpos) {
    return (a.window > 0 ? max(0, qpos - a.window + 1) : 0) / 64;
}
__device__ __forceinline__ bool decode_work(const AttnArgs& a, DecodeWork& w) {
    w.seq = a.chunk_seq[blockIdx.x];
    if (w.seq < 0) return false;
    w.split = a.chunk_idx[blockIdx.x];
    const int qpos = a.seq_pos0[w.seq];
    const int first = decode_first_page(a, qpos), end = qpos / 64 + 1;
    w.n_chunks = (end - first + a.pages_per_chunk - 1) / a.pages_per_chunk;
    w.page_lo = first + w.split * a.pages_per_chunk;
    w.page_hi = min(end, w.page_lo + a.pages_per_chunk);
    return true;
}
