// Arguments shared by the attention kernels over the paged cache.
#pragma once
#include <stdint.h>

#define NEG_BIG (-1e30f)

struct AttnArgs {
    const void* q;            // [T][H*d]
    const void* k_pages;      // [n_pages][G][PAGE][d]
    const void* v_pages;      // [n_pages][G][d][PAGE]
    void* out;                // [T][H*d]
    float* partial;           // decode split-K: [n_seq][H][n_splits][d+2], or null
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
    int n_splits;   // decode only
};
