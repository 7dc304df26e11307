// Row-wise kernels: embedding gather, RMSNorm, rotation + cache write, and the small
// element-wise helpers.  One workgroup handles one row (token); all arithmetic is float.
#include "common.h"
#include "api.h"
#include "attention.h"

// ---- embedding: x[t][:] = table[tokens[t]][:] ------------------------------------------
// picolm/model_core.c:1785-1786, :2758-2762: the row is converted to float, no scaling.
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int32_t* __restrict__ tokens,
                             float* __restrict__ x, int D, int V) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);      // ids are checked on the host; stay in bounds anyway
    const TW* row = table + (size_t)tok * D;
    float* out = x + (size_t)t * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) out[i] = to_f32<TW>(row[i]);
}

// out[i] = src[index[i]]: the tokens of the sequences that go on, picked from what a sampling kernel
// drew for a larger batch, without the host having seen them.
__global__ void gather_i32_kernel(int32_t* __restrict__ out, const int32_t* __restrict__ src, const int32_t* __restrict__ index, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = src[index[i]];
}

extern "C" int picolm_gather_i32(int32_t* out, const int32_t* src, const int32_t* index, int n, hipStream_t stream) {
    PICOLM_REQUIRE(out && src && index && n >= 0, "gather_i32: null argument");
    if (n == 0) return 0;
    gather_i32_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(out, src, index, n);
    PICOLM_LAUNCH_CHECK("gather_i32");
    return 0;
}

extern "C" int picolm_embed(const void* table, int table_dt, const int32_t* tokens, float* x,
                            int T, int D, int V, hipStream_t stream) {
    PICOLM_REQUIRE(T >= 0 && D > 0 && V > 0, "embed: bad sizes T=%d D=%d V=%d", T, D, V);
    if (T == 0) return 0;
    dim3 grid(T), block(256);
    if (table_dt == PICOLM_F32)
        embed_kernel<float><<<grid, block, 0, stream>>>((const float*)table, tokens, x, D, V);
    else if (table_dt == PICOLM_BF16)
        embed_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)table, tokens, x, D, V);
    else
        PICOLM_REQUIRE(false, "embed: unknown table dtype %d", table_dt);
    PICOLM_LAUNCH_CHECK("embed");
    return 0;
}

// ---- RMSNorm ---------------------------------------------------------------------------
// picolm/tensor.c:2942-3064: ss = sum x^2; r = 1/sqrtf(ss/size + eps); out = (x*r)*w.
// `rows` (optional) selects which rows of x are normed; output row i is dense.
#define NORM_THREADS 256
#define NORM_REGS 16        // a row of up to NORM_THREADS * 4 * NORM_REGS values stays in registers
template <typename TO>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_kernel(const float* __restrict__ x,
                                                               const float* __restrict__ w,
                                                               TO* __restrict__ out,
                                                               const int32_t* __restrict__ rows, int D,
                                                               float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float* xr = x + (size_t)r * D;
    TO* o = out + (size_t)i * D;
    float ss = 0.f;
    if (D % 4 == 0 && D <= NORM_THREADS * 4 * NORM_REGS) {
        // the row is read once, as float4, and kept
        float4 v[NORM_REGS], ww[NORM_REGS];
        const int nv = D / 4;
#pragma unroll
        for (int j = 0; j < NORM_REGS; ++j) {
            const int idx = threadIdx.x + j * NORM_THREADS;
            if (idx < nv) {
                v[j] = ((const float4*)xr)[idx];
                ww[j] = ((const float4*)w)[idx];         // asked for now: one trip to memory, not two
            }
        }
#pragma unroll
        for (int j = 0; j < NORM_REGS; ++j) {
            const int idx = threadIdx.x + j * NORM_THREADS;
            if (idx < nv) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
        }
        ss = block_sum(ss, scratch);
        const float scale = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
        for (int j = 0; j < NORM_REGS; ++j) {
            const int idx = threadIdx.x + j * NORM_THREADS;
            if (idx < nv) {
                // one store of four values (D % 4 == 0 and the rows of `out` are dense, so it is aligned)
                struct alignas(4 * sizeof(TO)) Four { TO a, b, c, d; };
                Four f = {from_f32<TO>((v[j].x * scale) * ww[j].x), from_f32<TO>((v[j].y * scale) * ww[j].y),
                          from_f32<TO>((v[j].z * scale) * ww[j].z), from_f32<TO>((v[j].w * scale) * ww[j].w)};
                ((Four*)o)[idx] = f;
            }
        }
        return;
    }
    for (int j = threadIdx.x; j < D; j += blockDim.x) {
        float v = xr[j];
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)D + eps);
    for (int j = threadIdx.x; j < D; j += blockDim.x) o[j] = from_f32<TO>((xr[j] * scale) * w[j]);
}

extern "C" int picolm_rmsnorm(const float* x, const float* w, void* out, int out_dt,
                              const int32_t* rows, int n_rows, int D, float eps,
                              hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && D > 0, "rmsnorm: bad sizes rows=%d D=%d", n_rows, D);
    PICOLM_REQUIRE(D % 4 != 0 || ((((uintptr_t)x | (uintptr_t)w) & 15) == 0 && ((uintptr_t)out & 15) == 0),
                   "rmsnorm: rows of a multiple of four values are read and written four at a time and must be 16-byte aligned");
    if (n_rows == 0) return 0;
    dim3 grid(n_rows), block(NORM_THREADS);
    if (out_dt == PICOLM_F32)
        rmsnorm_kernel<float><<<grid, block, 0, stream>>>(x, w, (float*)out, rows, D, eps);
    else if (out_dt == PICOLM_BF16)
        rmsnorm_kernel<bf16_t><<<grid, block, 0, stream>>>(x, w, (bf16_t*)out, rows, D, eps);
    else
        PICOLM_REQUIRE(false, "rmsnorm: unknown output dtype %d", out_dt);
    PICOLM_LAUNCH_CHECK("rmsnorm");
    return 0;
}

// ---- rotation of q and k, and the cache write of k and v ------------------------------------
// picolm rotates every q and k head of a token by its position's table row before k is
// cached and leaves v alone (picolm/model_core.c:1908, :2915; picolm/tensor.c:3216-3304).
// style 0: pairs (2i, 2i+1); style 1: pairs (i, i + d/2).  cos/sin == null: no rotation.
// q_out null: only keys and values are handled (the attention kernel that follows rotates q itself).
// A token's cache row is row pos % PAGE of physical page tok_page[t], which the host looked up
// in its copy of the page table: page_table[slot][(pos / PAGE) % ring_pages].
#define ROPE_HEADS 4
template <typename TC>
__global__ void rope_kv_store_kernel(const float* __restrict__ qkv, TC* __restrict__ q_out,
                                     TC* __restrict__ k_pages, TC* __restrict__ v_pages,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                     int style, const int32_t* __restrict__ tok_pos,
                                     const int32_t* __restrict__ tok_page, int H, int G, int d,
                                     const int32_t* __restrict__ rows, bool tiled, int head_first) {
    const int t = rows ? rows[blockIdx.x] : blockIdx.x;      // `rows`: the token rows this launch handles
    const int pos = tok_pos[t];
    const int half = d / 2;
    const float* row = qkv + (size_t)t * (H + 2 * G) * d;
    const float* c = cos_t ? cos_t + (size_t)pos * half : nullptr;
    const float* s = sin_t ? sin_t + (size_t)pos * half : nullptr;

    // keys are [page][G][PAGE][d]; values are kept transposed, [page][G][d][PAGE], so that the
    // attention kernels read eight consecutive keys of one column as one 16-byte chunk; within
    // a group's [PAGE][d] the order is that of k_page_offset / v_page_offset
    size_t page_base = 0;
    const int in_page = pos % PAGE_TOKENS;
    if (k_pages) page_base = ((size_t)tok_page[t] * G) * PAGE_TOKENS * d;
    // blockIdx.y takes ROPE_HEADS heads of the row: heads 0..H-1 are q, H..H+G-1 are k, then v.
    // A thread takes pair i of every head: all the heads' values are asked for before the first
    // is used, and a value head goes the same way as a key head without a rotation.
    const int head_lo = head_first + blockIdx.y * ROPE_HEADS, n_heads = H + 2 * G;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const int i0 = style == 0 ? 2 * i : i;
        const int i1 = style == 0 ? 2 * i + 1 : i + half;
        float x0[ROPE_HEADS], x1[ROPE_HEADS];
#pragma unroll
        for (int hh = 0; hh < ROPE_HEADS; ++hh) {
            const int head = min(head_lo + hh, n_heads - 1);
            x0[hh] = row[head * d + i0];
            x1[hh] = row[head * d + i1];
        }
        const float cc = c ? c[i] : 1.0f, ss = c ? s[i] : 0.0f;
#pragma unroll
        for (int hh = 0; hh < ROPE_HEADS; ++hh) {
            const int head = head_lo + hh;
            if (head >= n_heads) break;
            float y0 = x0[hh], y1 = x1[hh];
            if (c && head < H + G) {
                y0 = x0[hh] * cc - x1[hh] * ss;
                y1 = x0[hh] * ss + x1[hh] * cc;
            }
            if (head < H) {
                TC* q = q_out + (size_t)t * H * d + head * d;
                q[i0] = from_f32<TC>(y0);
                q[i1] = from_f32<TC>(y1);
            } else if (head < H + G) {
                if (k_pages) {
                    TC* k = k_pages + page_base + (size_t)(head - H) * PAGE_TOKENS * d;
                    k[k_page_offset(in_page, i0, d, tiled)] = from_f32<TC>(y0);
                    k[k_page_offset(in_page, i1, d, tiled)] = from_f32<TC>(y1);
                }
            } else if (v_pages) {
                TC* v = v_pages + page_base + (size_t)(head - H - G) * PAGE_TOKENS * d;
                v[v_page_offset(i0, in_page, d, tiled)] = from_f32<TC>(y0);
                v[v_page_offset(i1, in_page, d, tiled)] = from_f32<TC>(y1);
            }
        }
    }
}

// ---- keys and values of a prefill step into the cache, tile by tile --------------------------
// One workgroup takes one tile of a sequence's new tokens (the attention kernel's tiles: up to
// tile_tokens rows of one sequence) and one KV head.  Keys are rotated and written two pairs at a
// time.  Values are kept transposed, eight adjacent keys of a column in 16 bytes: where eight of
// the tile's tokens fill such a run (everywhere but at the two ends of a sequence's new tokens,
// and there too if they start at a multiple of eight) they are gathered and written as one
// chunk, else element by element.  q is left to the attention kernel.
template <typename TC> __device__ __forceinline__ void store_run(TC* p, const float* x, int n);
template <> __device__ __forceinline__ void store_run<float>(float* p, const float* x, int n) {
    for (int e = 0; e < n; e += 4) *(float4*)(p + e) = make_float4(x[e], x[e + 1], x[e + 2], x[e + 3]);
}
template <> __device__ __forceinline__ void store_run<bf16_t>(bf16_t* p, const float* x, int n) {
    for (int e = 0; e < n; e += 4) {
        uint2 v;
        v.x = (uint32_t)f32_to_bf16_bits(x[e]) | ((uint32_t)f32_to_bf16_bits(x[e + 1]) << 16);
        v.y = (uint32_t)f32_to_bf16_bits(x[e + 2]) | ((uint32_t)f32_to_bf16_bits(x[e + 3]) << 16);
        *(uint2*)(p + e) = v;
    }
}
template <typename TC>
__global__ __launch_bounds__(256) void kv_store_tiles_kernel(const float* __restrict__ qkv, TC* __restrict__ k_pages,
                                                             TC* __restrict__ v_pages, const float* __restrict__ cos_t,
                                                             const float* __restrict__ sin_t, int style,
                                                             const int32_t* __restrict__ tile_seq,
                                                             const int32_t* __restrict__ tile_q0, int tile_tokens,
                                                             const int32_t* __restrict__ seq_slot,
                                                             const int32_t* __restrict__ seq_pos0,
                                                             const int32_t* __restrict__ seq_nnew,
                                                             const int32_t* __restrict__ cu_seqlens,
                                                             const int32_t* __restrict__ page_table, int max_pages,
                                                             int ring_pages, int H, int G, int d, bool tiled) {
    const int tile = blockIdx.x, g = blockIdx.y;
    const int seq = tile_seq[tile], q0 = tile_q0[tile];
    const int n = min(tile_tokens, seq_nnew[seq] - q0);
    if (n <= 0) return;
    const int P0 = seq_pos0[seq] + q0;                       // position of the tile's first token
    const size_t stride = (size_t)(H + 2 * G) * d;
    const float* rows = qkv + ((size_t)cu_seqlens[seq] + q0) * stride;
    const float* kbase = rows + (size_t)(H + g) * d;
    const float* vbase = rows + (size_t)(H + G + g) * d;
    const int32_t* pt = page_table + (size_t)seq_slot[seq] * max_pages;
    const size_t page_elems = (size_t)G * PAGE_TOKENS * d, head_off = (size_t)g * PAGE_TOKENS * d;
    const int half = d / 2, quads = d / 4;                   // d is a multiple of 4 (the host sees to that)
    // (keys and values of a tile in workgroups of their own: twice the loads in flight)
    if (blockIdx.z == 0)
    for (int idx = threadIdx.x; idx < n * quads; idx += 256) {
        const int j = idx / quads, u = idx % quads;
        const int pos = P0 + j, key = pos % PAGE_TOKENS;
        const float* row = kbase + (size_t)j * stride;
        TC* k = k_pages + (size_t)pt[(pos / PAGE_TOKENS) % ring_pages] * page_elems + head_off;
        float c0 = 1.f, s0 = 0.f, c1 = 1.f, s1 = 0.f;
        if (cos_t) {
            const float2 cc = *(const float2*)(cos_t + (size_t)pos * half + 2 * u);
            const float2 ss = *(const float2*)(sin_t + (size_t)pos * half + 2 * u);
            c0 = cc.x, c1 = cc.y, s0 = ss.x, s1 = ss.y;
        }
        if (style == 0) {               // pairs (4u, 4u+1), (4u+2, 4u+3)
            const float4 x = *(const float4*)(row + 4 * u);
            const float y[4] = {x.x * c0 - x.y * s0, x.x * s0 + x.y * c0, x.z * c1 - x.w * s1, x.z * s1 + x.w * c1};
            store_run<TC>(k + k_page_offset(key, 4 * u, d, tiled), y, 4);
        } else {                        // pairs (2u, 2u + d/2), (2u+1, 2u+1 + d/2)
            const float2 lo = *(const float2*)(row + 2 * u), hi = *(const float2*)(row + half + 2 * u);
            TC* klo = k + k_page_offset(key, 2 * u, d, tiled);
            TC* khi = k + k_page_offset(key, half + 2 * u, d, tiled);
            klo[0] = from_f32<TC>(lo.x * c0 - hi.x * s0);
            klo[1] = from_f32<TC>(lo.y * c1 - hi.y * s1);
            khi[0] = from_f32<TC>(lo.x * s0 + hi.x * c0);
            khi[1] = from_f32<TC>(lo.y * s1 + hi.y * c1);
        }
    }
    if (blockIdx.z == 0) return;
    const int c_lo = P0 >> 3, n_runs = ((P0 + n - 1) >> 3) - c_lo + 1;      // runs of eight keys the tile touches
    for (int idx = threadIdx.x; idx < n_runs * d; idx += 256) {
        const int c = c_lo + idx / d, i = idx % d;
        const int k_lo = max(P0, 8 * c), k_hi = min(P0 + n, 8 * c + 8);
        TC* v = v_pages + (size_t)pt[(8 * c / PAGE_TOKENS) % ring_pages] * page_elems + head_off;
        const float* col = vbase + (size_t)(k_lo - P0) * stride + i;
        if (k_hi - k_lo == 8) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = col[(size_t)e * stride];
            store_run<TC>(v + v_page_offset(i, (8 * c) % PAGE_TOKENS, d, tiled), x, 8);
        } else {
            for (int key = k_lo; key < k_hi; ++key)
                v[v_page_offset(i, key % PAGE_TOKENS, d, tiled)] = from_f32<TC>(col[(size_t)(key - k_lo) * stride]);
        }
    }
}

extern "C" int picolm_kv_store_tiles(const float* qkv, void* k_pages, void* v_pages, int dt, const float* cos_t,
                                     const float* sin_t, int style, const int32_t* tile_seq, const int32_t* tile_q0,
                                     int n_tiles, int tile_tokens, const int32_t* seq_slot, const int32_t* seq_pos0,
                                     const int32_t* seq_nnew, const int32_t* cu_seqlens, const int32_t* page_table,
                                     int max_pages, int ring_pages, int H, int G, int d, hipStream_t stream) {
    PICOLM_REQUIRE(n_tiles >= 0 && tile_tokens > 0 && H > 0 && G > 0 && d > 0 && d % 4 == 0,
                   "kv_store_tiles: bad sizes tiles=%d of %d H=%d G=%d d=%d (d in multiples of 4)", n_tiles, tile_tokens, H, G, d);
    PICOLM_REQUIRE(max_pages > 0 && ring_pages > 0 && ring_pages <= max_pages, "kv_store_tiles: %d pages a row, a ring of %d", max_pages, ring_pages);
    PICOLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "kv_store_tiles: need both tables or none");
    PICOLM_REQUIRE(style == 0 || style == 1, "kv_store_tiles: unknown pairing %d", style);
    PICOLM_REQUIRE(qkv && k_pages && v_pages && ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)k_pages & 15) == 0 && ((uintptr_t)v_pages & 15) == 0,
                   "kv_store_tiles: the rows and the cache must be there, 16-byte aligned");
    if (n_tiles == 0) return 0;
    dim3 grid(n_tiles, G, 2), block(256);
    if (dt == PICOLM_F32)
        kv_store_tiles_kernel<float><<<grid, block, 0, stream>>>(qkv, (float*)k_pages, (float*)v_pages, cos_t, sin_t, style, tile_seq, tile_q0,
                                                                 tile_tokens, seq_slot, seq_pos0, seq_nnew, cu_seqlens, page_table,
                                                                 max_pages, ring_pages, H, G, d, kv_pages_tiled(dt, d));
    else if (dt == PICOLM_BF16)
        kv_store_tiles_kernel<bf16_t><<<grid, block, 0, stream>>>(qkv, (bf16_t*)k_pages, (bf16_t*)v_pages, cos_t, sin_t, style, tile_seq,
                                                                  tile_q0, tile_tokens, seq_slot, seq_pos0, seq_nnew, cu_seqlens,
                                                                  page_table, max_pages, ring_pages, H, G, d, kv_pages_tiled(dt, d));
    else
        PICOLM_REQUIRE(false, "kv_store_tiles: unknown dtype %d", dt);
    PICOLM_LAUNCH_CHECK("kv_store_tiles");
    return 0;
}

extern "C" int picolm_rope_kv_store(const float* qkv, void* q_out, void* k_pages, void* v_pages,
                                    int dt, const float* cos_t, const float* sin_t, int style,
                                    const int32_t* tok_pos, const int32_t* tok_page, int T, int H, int G,
                                    int d, const int32_t* rows, hipStream_t stream) {
    PICOLM_REQUIRE(T >= 0 && H > 0 && G > 0 && d > 0 && d % 2 == 0,
                   "rope_kv_store: bad sizes T=%d H=%d G=%d d=%d", T, H, G, d);
    PICOLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_kv_store: need both tables or none");
    PICOLM_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rope_kv_store: need both caches or none");
    PICOLM_REQUIRE(!k_pages || tok_page, "rope_kv_store: writing the cache needs every token's page");
    PICOLM_REQUIRE(style == 0 || style == 1, "rope_kv_store: unknown pairing %d", style);
    PICOLM_REQUIRE(q_out || k_pages, "rope_kv_store: neither q nor the cache to write");
    if (T == 0) return 0;
    const int head_first = q_out ? 0 : H;
    dim3 grid(T, ceil_div(H + 2 * G - head_first, ROPE_HEADS)), block(d / 2 >= 64 ? 64 : 32);
    if (dt == PICOLM_F32)
        rope_kv_store_kernel<float><<<grid, block, 0, stream>>>(
            qkv, (float*)q_out, (float*)k_pages, (float*)v_pages, cos_t, sin_t, style, tok_pos, tok_page,
            H, G, d, rows, kv_pages_tiled(dt, d), head_first);
    else if (dt == PICOLM_BF16)
        rope_kv_store_kernel<bf16_t><<<grid, block, 0, stream>>>(
            qkv, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, cos_t, sin_t, style, tok_pos, tok_page,
            H, G, d, rows, kv_pages_tiled(dt, d), head_first);
    else
        PICOLM_REQUIRE(false, "rope_kv_store: unknown dtype %d", dt);
    PICOLM_LAUNCH_CHECK("rope_kv_store");
    return 0;
}
