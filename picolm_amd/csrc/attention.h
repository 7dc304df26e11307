// Arguments shared by the attention kernels over the paged cache.
#pragma once
#include <stdint.h>

#define NEG_BIG (-1e30f)

struct AttnArgs {
    const void* q;            // [T][H*d]
    const void* k_pages;      // [n_pages][G][PAGE][d]     (within [PAGE][d] in the order of
    const void* v_pages;      // [n_pages][G][d][PAGE]      k_page_offset / v_page_offset)
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

// ---- the order of a page's elements ---------------------------------------------------------
// A page holds, per KV group, the keys K[64][d] and the values transposed V^T[d][64].  Pages of
// the vector-ALU kernels (32-bit, or head sizes the matrix-core kernels do not take) keep these
// as plain arrays.  Pages of the matrix-core kernels (bfloat16, d a multiple of 32 up to 256) keep their
// 16-byte chunks in the order in which a wave takes them as MFMA operands, so that every
// wave-wide load reads 1 KB of adjacent memory:
//   K   chunk ((tile * d/16 + kstep) * 64 + lane): key 32*tile + key_of_row(lane % 32),
//       elements 16*kstep + 8*(lane / 32) .. + 8
//   V^T chunk (((tile * d/32 + dblock) * 2 + step) * 64 + lane): row 32*dblock + lane % 32,
//       keys 32*tile + 16*step + 8*(lane / 32) .. + 8
// Row i of an S^T tile holds key_of_row(i) of the tile's 32 keys.  The accumulator of a lane in
// wave half h holds rows 8a + 4h + b (a = 0..3, b = 0..3) as element 4a + b; with this map they
// are the keys 8h .. 8h+7 (elements 0..7) and 16+8h .. 16+8h+7 (elements 8..15): P^T for step ks
// of the second MFMA is elements 8ks .. 8ks+7 as they are.
__host__ __device__ __forceinline__ int key_of_row(int i) {
    const int hh = (i >> 2) & 1, aa = i >> 3, bb = i & 3;
    return 16 * (aa >> 1) + 8 * hh + 4 * (aa & 1) + bb;
}
__host__ __device__ __forceinline__ int row_of_key(int k) {
    const int aa = 2 * (k >> 4) + ((k >> 2) & 1), hh = (k >> 3) & 1, bb = k & 3;
    return 8 * aa + 4 * hh + bb;
}
// whether pages of this dtype and head size are in the matrix-core kernels' order
__host__ __device__ __forceinline__ bool kv_pages_tiled(int dt, int d) {
    return dt == PICOLM_BF16 && d >= 32 && d <= 256 && d % 32 == 0;
}
// offset of K[key][i] and of V^T[i][key] within one group's part of a page
__host__ __device__ __forceinline__ int k_page_offset(int key, int i, int d, bool tiled) {
    if (!tiled) return key * d + i;
    const int chunk = i >> 3;
    return ((((key >> 5) * (d >> 4) + (chunk >> 1)) * 64 + (chunk & 1) * 32 + row_of_key(key & 31)) << 3) + (i & 7);
}
__host__ __device__ __forceinline__ int v_page_offset(int i, int key, int d, bool tiled) {
    if (!tiled) return i * PAGE_TOKENS + key;
    const int kc = key >> 3;      // eight keys: tile kc / 4, step (kc / 2) % 2, wave half kc % 2
    return (((((kc >> 2) * (d >> 5) + (i >> 5)) * 2 + ((kc >> 1) & 1)) * 64 + (kc & 1) * 32 + (i & 31)) << 3) + (key & 7);
}

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
    // The count of entries in use and this workgroup's entry are asked for together (the list has
    // room for every workgroup of the launch): one trip to memory, not two.  Workgroups past the
    // count leave at once.
    const int4* e = (const int4*)a.chunk_list + 2 * ((size_t)entry + 1);
    const int4 e0 = e[0], e1 = e[1];
    if (entry >= a.chunk_list[0]) return false;
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
