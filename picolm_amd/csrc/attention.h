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
    // decode: the step's work list, eight ints an entry.  Entry 0 is a header whose first int is
    // the number of entries in use; workgroup x takes entry 1 + x if x is below that number:
    // {sequence, which chunk of the sequence, position of the new token, cache slot,
    //  physical pages of the chunk's first four pages (-1 past its end)}
    const int32_t* chunk_list;
    int pages_per_chunk;
    int max_splits;             // chunks a sequence can have: stride of `partial`
    // decode with the rotation inside (matrix-core kernel only): q, and the new token's k and v,
    // are taken from the float rows qkv[n_seq][(H+2G)*d]; q and k are rotated by the tables
    // (cos_t null: no rotation), the new key and value join the attention from registers and are
    // written to row position % 64 of physical page tok_page[sequence]
    const float* qkv;
    const float* cos_t;
    const float* sin_t;
    const int32_t* tok_page;
    int rope_style;             // 0 pairs (2i, 2i+1), 1 pairs (i, i + d/2)
    // decode, matrix-core kernel: one counter per (sequence, workgroup of heads), zero between
    // launches.  With it the workgroup that finishes a sequence's last chunk combines the chunks
    // itself and no merge kernel runs; null: the merge kernel does.
    int32_t* chunks_done;
};

// What a decode workgroup has to do.  A sequence whose visible pages fit one chunk is finished by
// its workgroup; otherwise every chunk leaves (max, sum, acc) in `partial` and the merge kernel
// combines them.  The host's work list is built from the same arithmetic.  In a decode step row
// i of q and of the output belongs to sequence i.
struct DecodeWork {
    int seq, split, qpos, slot, page_lo, page_hi, n_chunks;
    int phys[4];
};
__device__ __forceinline__ int decode_first_page(int window, int qpos) {
    return (window > 0 ? max(0, qpos - window + 1) : 0) / 64;
}
// The decode grid is one-dimensional: workgroup b takes entry b / per_entry and is number
// b % per_entry (KV group, chunk of heads) of that entry's workgroups, so that all workgroups of
// entries in use are handed out before those that find nothing to do.
__device__ __forceinline__ bool decode_work(const AttnArgs& a, int per_entry, DecodeWork& w, int& which) {
    const int entry = blockIdx.x / per_entry;
    which = blockIdx.x % per_entry;
    // the count is one scalar load for the whole workgroup: those past it leave at once
    if (entry >= a.chunk_list[0]) return false;
    const int4* e = (const int4*)a.chunk_list + 2 * ((size_t)entry + 1);
    const int4 e0 = e[0], e1 = e[1];
    w.seq = e0.x;
    w.split = e0.y;
    w.qpos = e0.z;
    w.slot = e0.w;
    w.phys[0] = e1.x;
    w.phys[1] = e1.y;
    w.phys[2] = e1.z;
    w.phys[3] = e1.w;
    const int first = decode_first_page(a.window, w.qpos), end = w.qpos / 64 + 1;
    w.n_chunks = (end - first + a.pages_per_chunk - 1) / a.pages_per_chunk;
    w.page_lo = first + w.split * a.pages_per_chunk;
    w.page_hi = min(end, w.page_lo + a.pages_per_chunk);
    return true;
}
