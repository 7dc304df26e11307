// Attention over the paged cache on the vector ALU, for any head size up to 1,024 (a size that is
// no multiple of 16 leaves the last of a row's column groups partly empty; one above 256 goes
// through LDS in pieces of 256 columns), any number of heads and groups, float or bf16 storage.
// One kernel serves
// both kinds of step: a tile is up to 16 "rows" that share one KV head.
//   prefill: rows = consecutive new tokens of one sequence, for one query head;
//   decode : rows = the query heads of one KV group, for a sequence's single new token,
//            optionally over a slice of the pages (split-K) whose partial results a second
//            kernel merges.
// The recurrence is picolm's online softmax (picolm/model_attention.c:43-140): running
// maximum m, running sum l, accumulator rescaled by exp(m_old - m_new); key t is visible to
// a query at position p iff t <= p (and p - t < window when a window is set).
// picolm's split kernels keep (max, sum, acc) per split and merge with exp(m_i - M)
// (picolm/backend_gpu_kernels.cu:802-963); the same shape is used here.
#include "common.h"
#include "api.h"
#include "attention.h"

#define AT_ROWS 16
#define AT_THREADS 256
#define AT_MAX_D 1024
#define AT_CHUNK 256        // columns of a head that lie in LDS at a time: a larger head goes through in pieces


// MAXD: the largest head size of this instance (its accumulators are registers: MAXD / 16 a thread).
template <typename T, int MAXD>
__global__ __launch_bounds__(AT_THREADS) void attn_tile_kernel(AttnArgs a) {
    extern __shared__ float lds[];
    const int d = a.d;
    const int dl = min(d, AT_CHUNK), dp = dl + 1;
    const bool whole = d <= AT_CHUNK;           // the queries lie in LDS once and for all
    float* Qs = lds;                            // [AT_ROWS][dl]
    float* KVs = Qs + AT_ROWS * dl;             // [PAGE][dl+1]
    float* Ps = KVs + PAGE_TOKENS * dp;         // [AT_ROWS][PAGE]
    float* alpha_s = Ps + AT_ROWS * PAGE_TOKENS;  // [AT_ROWS]
    float* l_s = alpha_s + AT_ROWS;             // [AT_ROWS]
    float* m_s = l_s + AT_ROWS;                 // [AT_ROWS]
    __shared__ int row_tok[AT_ROWS], row_head[AT_ROWS], row_qpos[AT_ROWS];

    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int R = a.H / a.G;
    int seq, g, split = 0, n_rows;
    DecodeWork work = {};
    if (a.decode) {
        const int chunks = (R + AT_ROWS - 1) / AT_ROWS;
        int which;
        if (!decode_work(a, a.G * chunks, work, which)) return;
        seq = work.seq;
        split = work.split;
        g = which / chunks;
        const int chunk = which % chunks;
        n_rows = min(AT_ROWS, R - chunk * AT_ROWS);
        if (tid < AT_ROWS) {
            row_tok[tid] = seq;
            row_head[tid] = g * R + chunk * AT_ROWS + tid;
            row_qpos[tid] = work.qpos;
        }
    } else {
        seq = a.tile_seq[blockIdx.x];
        const int q0 = a.tile_q0[blockIdx.x];
        const int h = blockIdx.y;
        g = h / R;
        n_rows = min(AT_ROWS, a.seq_nnew[seq] - q0);
        if (tid < AT_ROWS) {
            row_tok[tid] = a.cu_seqlens[seq] + q0 + tid;
            row_head[tid] = h;
            row_qpos[tid] = a.seq_pos0[seq] + q0 + tid;
        }
    }
    __syncthreads();
    // visible key range of the tile: [lo, hi]
    const int qpos_first = row_qpos[0], qpos_last = row_qpos[n_rows - 1];
    const int hi = qpos_last;
    const int lo = a.window > 0 ? max(0, qpos_first - a.window + 1) : 0;
    int page_lo = lo / PAGE_TOKENS, page_hi = hi / PAGE_TOKENS + 1;   // [page_lo, page_hi)
    if (a.decode) {
        page_lo = work.page_lo;
        page_hi = work.page_hi;
    }

    const T* q = (const T*)a.q;
    // columns c0 .. c0 + dc of the tile's queries into LDS
    auto load_q = [&](int c0, int dc) {
        for (int idx = tid; idx < AT_ROWS * dc; idx += AT_THREADS) {
            const int r = idx / dc, c = idx % dc;
            Qs[r * dl + c] = r < n_rows ? to_f32<T>(q[(size_t)row_tok[r] * a.H * d + (size_t)row_head[r] * d + c0 + c]) : 0.f;
        }
    };
    if (whole) load_q(0, d);
    // per-wave running statistics of its 4 rows (uniform across the wave)
    float m_run[4], l_run[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        m_run[i] = NEG_BIG;
        l_run[i] = 0.f;
    }
    // PV ownership: thread -> (row pr, column group pc), columns pc + 16*j
    const int pr = tid / 16, pc = tid % 16;
    const int n_cg = pc < d ? (d - pc + 15) / 16 : 0;      // this thread's columns pc + 16*j below d
    float acc[MAXD / 16];
#pragma unroll
    for (int j = 0; j < MAXD / 16; ++j) acc[j] = 0.f;

    const int slot = a.decode ? work.slot : a.seq_slot[seq];
    const int32_t* pt = a.page_table + (size_t)slot * a.max_pages;
    const size_t page_elems = (size_t)a.G * PAGE_TOKENS * d;

    for (int page = page_lo; page < page_hi; ++page) {
        const int phys = pt[page % a.ring_pages];
        const size_t base = (size_t)phys * page_elems + (size_t)g * PAGE_TOKENS * d;
        const int key0 = page * PAGE_TOKENS;
        const int n_keys = min(PAGE_TOKENS, hi - key0 + 1);   // rows beyond are not this sequence's
        // scores: wave handles rows 4*wave .. +3, lane = key; a head wider than the chunk adds up piece by piece
        float s[4] = {0.f, 0.f, 0.f, 0.f};
        for (int c0 = 0; c0 < d; c0 += AT_CHUNK) {
            const int dc = min(AT_CHUNK, d - c0);
            __syncthreads();                                   // whoever read KVs, Qs or Ps before is done
            if (!whole) load_q(c0, dc);
            const T* kp = (const T*)a.k_pages + base;
            for (int idx = tid; idx < PAGE_TOKENS * dc; idx += AT_THREADS) {
                const int r = idx / dc, c = idx % dc;
                KVs[r * dp + c] = r < n_keys ? to_f32<T>(kp[(size_t)r * d + c0 + c]) : 0.f;
            }
            __syncthreads();
            const float* kr = KVs + lane * dp;
            const float* q0p = Qs + (4 * wave) * dl;
            for (int c = 0; c < dc; ++c) {
                const float kv = kr[c];
#pragma unroll
                for (int i = 0; i < 4; ++i) s[i] = fmaf(q0p[i * dl + c], kv, s[i]);
            }
        }
        {
            const int kpos = key0 + lane;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 4 * wave + i;
                const int qp = row_qpos[r];
                const bool vis = r < n_rows && kpos <= qp && (a.window <= 0 || qp - kpos < a.window);
                const float sc = vis ? s[i] * a.scale : NEG_BIG;
                const float m_new = fmaxf(m_run[i], wave_max(sc));
                const float p = vis ? expf(sc - m_new) : 0.f;
                const float al = expf(m_run[i] - m_new);
                l_run[i] = l_run[i] * al + wave_sum(p);
                m_run[i] = m_new;
                Ps[r * PAGE_TOKENS + lane] = p;
                if (lane == 0) alpha_s[r] = al;
            }
        }
        __syncthreads();
        const float al = alpha_s[pr];
#pragma unroll
        for (int j = 0; j < MAXD / 16; ++j) acc[j] *= al;
#pragma unroll
        for (int ci = 0; ci < MAXD / AT_CHUNK; ++ci) {
            const int c0 = ci * AT_CHUNK;
            if (c0 >= d) break;
            const int dc = min(AT_CHUNK, d - c0);
            if (ci > 0) __syncthreads();                       // the piece before has been used
            const T* vp = (const T*)a.v_pages + base + (size_t)c0 * PAGE_TOKENS;       // transposed: [d][PAGE]
            for (int idx = tid; idx < PAGE_TOKENS * dc; idx += AT_THREADS) {
                const int c = idx / PAGE_TOKENS, r = idx % PAGE_TOKENS;
                KVs[r * dp + c] = r < n_keys ? to_f32<T>(vp[idx]) : 0.f;
            }
            __syncthreads();
            const float* p = Ps + pr * PAGE_TOKENS;
            const int n_here = pc < dc ? (dc - pc + 15) / 16 : 0;      // this thread's columns of the piece
            for (int key = 0; key < n_keys; ++key) {
                const float pk = p[key];
                const float* vr = KVs + key * dp + pc;
#pragma unroll
                for (int j = 0; j < AT_CHUNK / 16; ++j)
                    if (j < n_here) acc[ci * (AT_CHUNK / 16) + j] = fmaf(pk, vr[16 * j], acc[ci * (AT_CHUNK / 16) + j]);
            }
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            l_s[4 * wave + i] = l_run[i];
            m_s[4 * wave + i] = m_run[i];
        }
    }
    __syncthreads();
    if (pr >= n_rows) return;
    const int tok = row_tok[pr], head = row_head[pr];
    if (a.decode && work.n_chunks > 1) {
        float* po = a.partial + (((size_t)seq * a.H + head) * a.max_splits + split) * (d + 2);
        if (pc == 0) {
            po[0] = m_s[pr];
            po[1] = l_s[pr];
        }
#pragma unroll
        for (int j = 0; j < MAXD / 16; ++j)
            if (j < n_cg) po[2 + pc + 16 * j] = acc[j];
    } else {
        const float l = l_s[pr];
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        T* o = (T*)a.out + (size_t)tok * a.H * d + (size_t)head * d;
#pragma unroll
        for (int j = 0; j < MAXD / 16; ++j)
            if (j < n_cg) o[pc + 16 * j] = from_f32<T>(acc[j] * inv);
    }
}

// out = sum_i exp(m_i - M) acc_i / sum_i exp(m_i - M) l_i over the splits of one (seq, head).
// One wave per (seq, head): lanes take splits for the statistics, then columns for the sum.
#define MERGE_WAVES 4
template <typename T>
__global__ __launch_bounds__(MERGE_WAVES * WAVE) void attn_merge_kernel(AttnArgs a, int n_units) {
    const int unit = blockIdx.x * MERGE_WAVES + threadIdx.x / WAVE;
    const int lane = threadIdx.x % WAVE;
    if (unit >= n_units) return;
    const int H = a.H, d = a.d;
    const int seq = unit / H, head = unit % H;
    const int qpos = a.seq_pos0[seq];
    const int n_splits = (qpos / 64 + 1 - decode_first_page(a.window, qpos) + a.pages_per_chunk - 1) / a.pages_per_chunk;
    if (n_splits <= 1) return;                         // its one workgroup wrote the result itself
    const int stride = d + 2;
    const float* p = a.partial + (size_t)unit * a.max_splits * stride;
    // the first splits' columns are asked for together with the statistics, so that the sum
    // does not wait for a second trip to memory
    constexpr int EARLY = 8;
    float early[EARLY][4];
#pragma unroll
    for (int i = 0; i < EARLY; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + j * WAVE;
            early[i][j] = (i < n_splits && c < d) ? p[(size_t)i * stride + 2 + c] : 0.f;
        }
    float m = NEG_BIG;
    for (int i = lane; i < n_splits; i += WAVE) m = fmaxf(m, p[(size_t)i * stride]);
    const float M = wave_max(m);
    float l = 0.f;
    for (int i = lane; i < n_splits; i += WAVE) l += expf(p[(size_t)i * stride] - M) * p[(size_t)i * stride + 1];
    const float L = wave_sum(l);
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    T* o = (T*)a.out + (size_t)seq * H * d + (size_t)head * d;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = lane + j * WAVE;
        if (c >= d) break;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < EARLY; ++i)
            if (i < n_splits) acc += expf(p[(size_t)i * stride] - M) * early[i][j];
        for (int i = EARLY; i < n_splits; ++i) acc += expf(p[(size_t)i * stride] - M) * p[(size_t)i * stride + 2 + c];
        o[c] = from_f32<T>(acc * inv);
    }
    for (int c = lane + 4 * WAVE; c < d; c += WAVE) {       // a head wider than 256
        float acc = 0.f;
        for (int i = 0; i < n_splits; ++i) acc += expf(p[(size_t)i * stride] - M) * p[(size_t)i * stride + 2 + c];
        o[c] = from_f32<T>(acc * inv);
    }
}

static size_t attn_lds_bytes(int d) {
    const int dl = d < AT_CHUNK ? d : AT_CHUNK;
    return sizeof(float) * ((size_t)AT_ROWS * dl + (size_t)PAGE_TOKENS * (dl + 1) + AT_ROWS * PAGE_TOKENS + 3 * AT_ROWS);
}

template <typename T, int MAXD>
static int launch_attn_sized(const AttnArgs& a, dim3 grid, hipStream_t stream) {
    const size_t lds = attn_lds_bytes(a.d);
    static size_t raised = 48 * 1024;      // what a kernel may use without asking
    if (lds > raised) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_tile_kernel<T, MAXD>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        PICOLM_REQUIRE(e == hipSuccess, "attention: cannot raise the LDS limit to %zu: %s", lds,
                       hipGetErrorString(e));
        raised = lds;
    }
    attn_tile_kernel<T, MAXD><<<grid, dim3(AT_THREADS), lds, stream>>>(a);
    PICOLM_LAUNCH_CHECK("attention");
    return 0;
}

// (heads of up to 256 have the kernel with 16 accumulators a thread, wider ones that with 64)
template <typename T>
static int launch_attn(const AttnArgs& a, dim3 grid, hipStream_t stream) {
    return a.d <= AT_CHUNK ? launch_attn_sized<T, AT_CHUNK>(a, grid, stream) : launch_attn_sized<T, AT_MAX_D>(a, grid, stream);
}

int check_decode_chunks(const char* who, const float* partial, const int32_t* chunk_list, int n_chunks,
                        int pages_per_chunk, int max_splits) {
    PICOLM_REQUIRE(chunk_list && n_chunks >= 0, "%s: needs the step's work list", who);
    PICOLM_REQUIRE(((uintptr_t)chunk_list & 15) == 0, "%s: the work list must be 16-byte aligned", who);
    PICOLM_REQUIRE(pages_per_chunk >= 1 && max_splits >= 1, "%s: bad chunking (%d pages a chunk, %d chunks a sequence)", who,
                   pages_per_chunk, max_splits);
    PICOLM_REQUIRE(max_splits == 1 || partial != nullptr, "%s: several chunks a sequence need a partial buffer", who);
    return 0;
}

static int check_attn_sizes(const char* who, int H, int G, int d, int max_pages, int ring_pages) {
    PICOLM_REQUIRE(H > 0 && G > 0 && H % G == 0, "%s: %d heads do not split over %d groups", who, H, G);
    PICOLM_REQUIRE(d >= 1 && d <= AT_MAX_D, "%s: head size %d is not in [1, %d]", who, d, AT_MAX_D);
    PICOLM_REQUIRE(max_pages > 0 && ring_pages > 0 && ring_pages <= max_pages,
                   "%s: bad page table geometry max_pages=%d ring_pages=%d", who, max_pages, ring_pages);
    return 0;
}

int picolm_attn_merge_launch(const AttnArgs& a, int dt, int n_seq, hipStream_t stream) {
    const int n_units = n_seq * a.H;
    dim3 mgrid(ceil_div(n_units, MERGE_WAVES)), mblock(MERGE_WAVES * WAVE);
    if (dt == PICOLM_F32) attn_merge_kernel<float><<<mgrid, mblock, 0, stream>>>(a, n_units);
    else attn_merge_kernel<bf16_t><<<mgrid, mblock, 0, stream>>>(a, n_units);
    PICOLM_LAUNCH_CHECK("attn_merge");
    return 0;
}

extern "C" int picolm_attn_prefill_generic(const void* q, const void* k_pages, const void* v_pages,
                                           void* out, int dt, const int32_t* tile_seq,
                                           const int32_t* tile_q0, int n_tiles,
                                           const int32_t* seq_slot, const int32_t* seq_pos0,
                                           const int32_t* seq_nnew, const int32_t* cu_seqlens,
                                           const int32_t* page_table, int max_pages, int ring_pages,
                                           int H, int G, int d, int window, float scale,
                                           hipStream_t stream) {
    if (check_attn_sizes("attn_prefill", H, G, d, max_pages, ring_pages)) return -1;
    PICOLM_REQUIRE(!kv_pages_tiled(dt, d), "attn_prefill: bfloat16 pages of head size %d are in the matrix-core kernels' order", d);
    PICOLM_REQUIRE(H <= 65535, "attn_prefill: %d heads exceed the grid", H);
    if (n_tiles <= 0) return 0;
    AttnArgs a = {q, k_pages, v_pages, out, nullptr, tile_seq, tile_q0, seq_slot, seq_pos0, seq_nnew,
                  cu_seqlens, page_table, max_pages, ring_pages, H, G, d, window, scale, 0, nullptr, 0, 1,
                  nullptr, nullptr, nullptr, nullptr, 0};
    dim3 grid(n_tiles, H);
    if (dt == PICOLM_F32) return launch_attn<float>(a, grid, stream);
    if (dt == PICOLM_BF16) return launch_attn<bf16_t>(a, grid, stream);
    PICOLM_REQUIRE(false, "attn_prefill: unknown dtype %d", dt);
}

extern "C" int picolm_attn_prefill_tile_rows(void) { return AT_ROWS; }

extern "C" int picolm_attn_decode_generic(const void* q, const void* k_pages, const void* v_pages,
                                          void* out, float* partial, int dt, int n_seq,
                                          const int32_t* chunk_list, int n_chunks, int pages_per_chunk,
                                          int max_splits, const int32_t* seq_pos0, const int32_t* page_table,
                                          int max_pages, int ring_pages, int H, int G, int d, int window,
                                          float scale, hipStream_t stream) {
    if (check_attn_sizes("attn_decode", H, G, d, max_pages, ring_pages)) return -1;
    PICOLM_REQUIRE(!kv_pages_tiled(dt, d), "attn_decode: bfloat16 pages of head size %d are in the matrix-core kernels' order", d);
    if (check_decode_chunks("attn_decode", partial, chunk_list, n_chunks, pages_per_chunk, max_splits)) return -1;
    PICOLM_REQUIRE(dt == PICOLM_F32 || dt == PICOLM_BF16, "attn_decode: unknown dtype %d", dt);
    if (n_seq <= 0 || n_chunks <= 0) return 0;
    const int chunks = ceil_div(H / G, AT_ROWS);
    PICOLM_REQUIRE((int64_t)n_chunks * G * chunks < (1ll << 31), "attn_decode: %d chunks of %d workgroups exceed the grid", n_chunks, G * chunks);
    AttnArgs a = {q, k_pages, v_pages, out, partial, nullptr, nullptr, nullptr, seq_pos0, nullptr, nullptr,
                  page_table, max_pages, ring_pages, H, G, d, window, scale, 1, chunk_list, pages_per_chunk, max_splits,
                  nullptr, nullptr, nullptr, nullptr, 0};
    dim3 grid(n_chunks * G * chunks);
    const int rc = dt == PICOLM_F32 ? launch_attn<float>(a, grid, stream) : launch_attn<bf16_t>(a, grid, stream);
    if (rc) return rc;
    return max_splits > 1 ? picolm_attn_merge_launch(a, dt, n_seq, stream) : 0;
}

// The order of a page's elements, for code that fills or reads pages on the host: offsets of
// K[key][i] (k_idx[key * d + i]) and of V^T[i][key] (v_idx[i * 64 + key]) within a group's part
// of a page of this dtype and head size.
extern "C" int picolm_kv_page_order(int dt, int d, int32_t* k_idx, int32_t* v_idx) {
    PICOLM_REQUIRE(d > 0 && k_idx && v_idx, "kv_page_order: bad arguments");
    const bool tiled = kv_pages_tiled(dt, d);
    for (int key = 0; key < PAGE_TOKENS; ++key)
        for (int i = 0; i < d; ++i) {
            k_idx[key * d + i] = k_page_offset(key, i, d, tiled);
            v_idx[i * PAGE_TOKENS + key] = v_page_offset(i, key, d, tiled);
        }
    return 0;
}
