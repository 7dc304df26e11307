// The engine of engine.h: host code only.  It keeps the books of the cache (slots, pages, page
// tables), plans every step (index arrays, the decode attention's work list, the prefill's tiles),
// walks the model's launch program through the library's kernel entry points, records decode
// steps as HIP graphs, and runs the generation loop.
#include "common.h"
#include "api.h"
#include "engine.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#define E_REQUIRE(code, cond, ...)            \
    do {                                      \
        if (!(cond)) {                        \
            picolm_set_error(__VA_ARGS__);    \
            return code;                      \
        }                                     \
    } while (0)
#define HIP_TRY(call)                                                              \
    do {                                                                           \
        hipError_t e__ = (call);                                                   \
        if (e__ != hipSuccess) {                                                   \
            picolm_set_error("%s: %s", #call, hipGetErrorString(e__));             \
            return PICOLM_ERR_DEVICE;                                              \
        }                                                                          \
    } while (0)
#define TRY(call)                 \
    do {                          \
        const int rc__ = (call);  \
        if (rc__) return rc__;    \
    } while (0)

static inline int pages_for(int64_t n_tokens) { return (int)((n_tokens + PAGE_TOKENS - 1) / PAGE_TOKENS); }
static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline int dt_bytes(int dt) { return dt == PICOLM_F32 ? 4 : 2; }

// ---- books: which pages are free, which slot holds which pages ---------------------------------
// picolm has one sequence and no slots (its "reset" is a memset, picolm/picolm.c:1391-1392).
struct PagePool {
    int n_pages = 0;
    std::vector<int> free_;      // pop_back hands out low numbers first
    std::vector<char> taken;
    void init(int n) {
        n_pages = n;
        free_.resize(n);
        for (int i = 0; i < n; ++i) free_[i] = n - 1 - i;
        taken.assign(n, 0);
    }
    int n_free() const { return (int)free_.size(); }
    void take(int n, std::vector<int>& out) {      // the caller has checked n <= n_free()
        for (int i = 0; i < n; ++i) {
            const int p = free_.back();
            free_.pop_back();
            taken[p] = 1;
            out.push_back(p);
        }
    }
    void give(const std::vector<int>& pages) {
        for (int p : pages) {
            taken[p] = 0;
            free_.push_back(p);
        }
    }
};

struct SlotTable {
    int n_slots = 0;
    std::vector<int> free_;
    std::vector<char> live;
    std::vector<int> length;
    void init(int n) {
        n_slots = n;
        free_.resize(n);
        for (int i = 0; i < n; ++i) free_[i] = n - 1 - i;
        live.assign(n, 0);
        length.assign(n, 0);
    }
    bool is_live(int s) const { return s >= 0 && s < n_slots && live[s]; }
};

// New tokens of one sequence that a group with a window takes in at once: its ring holds a window
// and one such chunk, so a longer prompt is written and answered chunk by chunk.
static const int WINDOW_STEP_TOKENS = 256;

struct KVGroup {
    picolm_kv_group spec;
    int max_pages = 0, ring_pages = 0, n_pages = 0;
    PagePool pool;
    std::vector<std::vector<int>> pages;     // slot -> its pages in logical order (a ring: page j lies at j % ring_pages)
    std::vector<int32_t> table_host;         // [n_slots][max_pages]
    int32_t* table_dev = nullptr;
    char* k = nullptr;                       // [n_entries][n_pages][G][64][d]
    char* v = nullptr;                       // [n_entries][n_pages][G][dv][64]
    size_t k_entry_bytes = 0, v_entry_bytes = 0;
    std::vector<int> dirty;                  // slots whose table row changed since the last flush
    int value_dim() const { return spec.v_head_dim ? spec.v_head_dim : spec.head_dim; }
    bool is_ring() const { return ring_pages < max_pages; }
    int need(int n_tokens) const { return std::min(pages_for(n_tokens), ring_pages); }
    int missing(int slot, int n_tokens) const { return std::max(0, need(n_tokens) - (int)pages[slot].size()); }
    // the first page that a query at `pos` sees
    int first_page(int pos) const { return spec.window > 0 ? std::max(0, pos - spec.window + 1) / PAGE_TOKENS : 0; }
};

struct StateGroup {
    picolm_state_group spec;
    char* data = nullptr;                    // [n_entries][n_slots][bytes_per_slot]
};

// ---- pinned staging for small uploads -------------------------------------------------------
// A ring in pinned host memory.  A region is handed out again only after the copy that read it
// has run (an event per region), so that no upload makes the host wait for the GPU's other work.
struct Stager {
    char* base = nullptr;
    size_t cap = 0, head = 0;
    struct Fence {
        size_t begin, end;
        hipEvent_t ev;
    };
    std::deque<Fence> fences;
    std::vector<hipEvent_t> spare;

    int drain() {
        for (auto& f : fences) {
            HIP_TRY(hipEventSynchronize(f.ev));
            spare.push_back(f.ev);
        }
        fences.clear();
        return 0;
    }
    int take(size_t bytes, void** out) {
        bytes = align_up(std::max<size_t>(bytes, 64), 64);
        if (bytes * 4 > cap) {
            TRY(drain());
            if (base) HIP_TRY(hipHostFree(base));
            base = nullptr;
            cap = align_up(bytes * 8, 1 << 16);
            HIP_TRY(hipHostMalloc((void**)&base, cap, hipHostMallocDefault));
            head = 0;
        }
        if (head + bytes > cap) head = 0;
        for (size_t i = 0; i < fences.size();) {
            if (fences[i].begin < head + bytes && head < fences[i].end) {
                HIP_TRY(hipEventSynchronize(fences[i].ev));
                spare.push_back(fences[i].ev);
                fences.erase(fences.begin() + i);
            } else {
                ++i;
            }
        }
        *out = base + head;
        return 0;
    }
    // the copy from the region taken last has been queued on `stream`
    int commit(size_t bytes, hipStream_t stream) {
        bytes = align_up(std::max<size_t>(bytes, 64), 64);
        hipEvent_t ev;
        if (!spare.empty()) {
            ev = spare.back();
            spare.pop_back();
        } else {
            HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        }
        HIP_TRY(hipEventRecord(ev, stream));
        fences.push_back({head, head + bytes, ev});
        head += bytes;
        return 0;
    }
    int upload(void* dst_dev, const void* src, size_t bytes, hipStream_t stream) {
        if (bytes == 0) return 0;
        void* p = nullptr;
        TRY(take(bytes, &p));
        memcpy(p, src, bytes);
        HIP_TRY(hipMemcpyAsync(dst_dev, p, bytes, hipMemcpyHostToDevice, stream));
        return commit(bytes, stream);
    }
    void destroy() {
        for (auto& f : fences) {
            (void)hipEventSynchronize(f.ev);
            (void)hipEventDestroy(f.ev);
        }
        for (auto ev : spare) (void)hipEventDestroy(ev);
        if (base) (void)hipHostFree(base);
        base = nullptr;
    }
};

// ---- a step's index arrays ---------------------------------------------------------------------
struct Span {
    int off = 0, n = 0;
};
struct TileList {
    int rows_per_tile = 0;
    Span seq, q0;
    int n = 0;
};
struct DecodeList {
    Span span;              // header entry and entries, eight ints each
    int n_chunks = 0;       // entries the launch covers
    int most = 1;           // chunks a sequence can have: stride of the partial results
};
// A slice of a prefill step along positions (new tokens lo .. lo + 255 of every sequence that has
// them): it looks like a step of its own to the attention kernels.
struct WindowChunk {
    int n_seq = 0, n_rows = 0;
    Span seq_slot, seq_pos0, seq_nnew, first_row, rows;
    std::vector<TileList> tiles;
    const TileList* tiles_of(int rows_per_tile) const {
        for (auto& t : tiles)
            if (t.rows_per_tile == rows_per_tile) return &t;
        return nullptr;
    }
};

// What the operations read of a step: sizes, and where each array lies in the int block.
struct StepPlan {
    int n_seq = 0, T = 0, n_want = 0, max_new = 0;
    bool is_decode = false, every_row = false;
    std::vector<int> slots, pos0, n_new;
    Span seq_slot, seq_pos0, seq_nnew, cu_seqlens, tok_pos, tok_seq, tokens, want_rows;
    std::vector<Span> write_pages;        // per KV group (n = 0: not needed)
    std::vector<DecodeList> lists;        // per KV group, decode steps
    std::vector<TileList> tiles;          // prefill steps
    std::vector<WindowChunk> window_chunks;   // prefill steps of more than WINDOW_STEP_TOKENS a sequence, where a group keeps a ring
    int pages_per_chunk = 0;
    std::vector<int32_t> ints;            // the host's copy of the block
    const int32_t* dev = nullptr;         // the block on the device
    int take(int n) {
        const int off = (int)ints.size();
        ints.resize(off + (n + 3) / 4 * 4, 0);     // what follows is read 16 bytes at a time
        return off;
    }
    const int32_t* at(const Span& s) const { return dev + s.off; }
    const TileList* tiles_of(int rows) const {
        for (auto& t : tiles)
            if (t.rows_per_tile == rows) return &t;
        return nullptr;
    }
};

// Pages that one workgroup of the decode attention takes: the largest of 4, 8, 16, 32, 64 within
// `max_pages_per_chunk` (what the kernel that will run was measured with) that still leaves
// `min_blocks` workgroups for the launch, which is most of the CUs; 4 (a page for each of four
// waves) if none does.  Fewer, larger chunks mean fewer partial results to merge and longer
// streams a wave (contexts of 16,000 tokens at batch 8: 6.03 ms a step with 64 pages, 6.24 with 16).
static int decode_pages_per_chunk(const std::vector<int>& pos0, int blocks_per_chunk, int max_pages_per_chunk) {
    const int min_blocks = 160;
    for (int ppc : {64, 32, 16, 8}) {
        if (ppc > max_pages_per_chunk) continue;
        int64_t chunks = 0;
        for (int p : pos0) chunks += (p / PAGE_TOKENS + 1 + ppc - 1) / ppc;
        if (chunks * std::max(1, blocks_per_chunk) >= min_blocks) return ppc;
    }
    return 4;
}

// The work list of a decode step over one group's pages: every sequence's visible pages (those of
// its last `window` keys, or all) cut into runs of `ppc`; an entry is {sequence, which chunk,
// position of the new token, slot, physical pages of the chunk's first four pages or -1}.  The
// chunks with the most pages come first: workgroups are handed out in the list's order, and the
// short last chunks then fill the gaps at the end.
// Returns the number of entries written behind the header at `out`; *most: chunks of the longest.
static int chunks_of(const KVGroup& g, int pos, int ppc) { return (pos / PAGE_TOKENS + 1 - g.first_page(pos) + ppc - 1) / ppc; }

static int fill_chunk_list(int32_t* out, const std::vector<int>& slots, const std::vector<int>& pos0, int ppc,
                           const KVGroup& g, int* most) {
    struct Chunk {
        int seq, idx, n_pages;
    };
    std::vector<Chunk> chunks;
    int longest = 0;
    for (int i = 0; i < (int)slots.size(); ++i) {
        const int first = g.first_page(pos0[i]), end = pos0[i] / PAGE_TOKENS + 1;
        const int n = (end - first + ppc - 1) / ppc;
        longest = std::max(longest, n);
        for (int c = 0; c < n; ++c) chunks.push_back({i, c, std::min(end - first - c * ppc, ppc)});
    }
    std::stable_sort(chunks.begin(), chunks.end(), [](const Chunk& a, const Chunk& b) { return a.n_pages > b.n_pages; });
    out[0] = (int)chunks.size();
    for (int j = 1; j < 8; ++j) out[j] = 0;
    for (size_t x = 0; x < chunks.size(); ++x) {
        const Chunk& c = chunks[x];
        int32_t* e = out + 8 * (x + 1);
        const int slot = slots[c.seq], first = g.first_page(pos0[c.seq]), end = pos0[c.seq] / PAGE_TOKENS + 1;
        e[0] = c.seq;
        e[1] = c.idx;
        e[2] = pos0[c.seq];
        e[3] = slot;
        for (int w = 0; w < 4; ++w) {
            const int page = first + c.idx * ppc + w;
            const bool inside = page < end && w < ppc;
            e[4 + w] = inside ? g.table_host[(size_t)slot * g.max_pages + page % g.ring_pages] : -1;
        }
    }
    *most = longest;
    return (int)chunks.size();
}

// A decode step (one new token per sequence, every row's logits wanted) over a block that stays
// in place, so that the step's launches can be recorded once and replayed: only the contents of
// the block change from step to step.
struct DecodeBatch {
    StepPlan plan;
    int32_t* dev = nullptr;
    int32_t* pinned[2] = {nullptr, nullptr};
    hipEvent_t sent[2] = {nullptr, nullptr};
    bool sent_once[2] = {false, false};
    int turn = 0;
    std::vector<int> live;             // per group: entries in use
    int64_t cache_version = -1;
    bool filled = false;
};

// ---- workspace -------------------------------------------------------------------------------
struct Workspace {
    char* base = nullptr;
    size_t cap = 0;
    int32_t* counters = nullptr;       // zero between launches (the kernels leave them so)
    std::vector<size_t> offsets;       // program buffers
    size_t prep_h[2] = {0, 0}, prep_ssq[2] = {0, 0}, partial = 0;
    int for_T = -1, for_want = -1, for_seq = -1, for_most = -1;
    int flip = 1;
    int64_t generation = 0;            // moves when the memory does
};

struct Prepared {                      // a norm that the product before has prepared
    const picolm_op* by = nullptr;
    const void* x = nullptr;
    const float* w = nullptr;
    float eps = 0.f;
    void* h = nullptr;
    float* ssq = nullptr;
    int parts = 0;
};

// A decode step of one shape (sequences, pages a chunk, chunks a sequence): its block, and the
// recording of its launches once it has been used twice.  All of them share one workspace (they
// run on one stream, one after the other); a recording holds that workspace's addresses and is
// dropped when it moves.
struct DecodeGraph {
    DecodeBatch batch;
    hipGraphExec_t exec = nullptr;
    int64_t ws_generation = -1;
    int uses = 0;
    int64_t last_used = 0;
};
static const size_t MAX_DECODE_SHAPES = 48;      // blocks and recordings kept; the least recently used goes first

struct picolm_engine {
    int dtype = PICOLM_BF16, vocab = 0, flags = 0;
    std::vector<picolm_op> ops;
    std::vector<picolm_buffer> buffers;
    int logits_buffer = -1;
    int max_seq_len = 0, max_pages = 0, n_slots = 0;
    SlotTable slots;
    std::vector<KVGroup> kv;
    std::vector<StateGroup> state;
    int64_t version = 0;
    size_t device_bytes = 0;
    // what the attention operations need of a step's plan
    std::vector<char> group_written;       // per group: some operation writes it
    std::vector<char> group_attended;      // per group: some operation attends over it
    std::vector<int> tile_rows;            // tile heights of the prefill kernels in use
    int decode_blocks_per_chunk = 1, decode_max_pages_per_chunk = 64;
    int counters_needed = 0;
    bool recordable = true;                // every called operation says that its launches may be recorded
    bool call_on_ring = false;             // a called operation uses a cache group that keeps a ring of pages
    size_t partial_floats_per_seq_chunk = 0;   // max over attention operations of H * (d + 2)
    int prep_n = 0;                        // widest output that prepares a norm
    // the running step
    StepPlan plan;                         // steps that are not recorded
    int32_t* plan_dev = nullptr;
    size_t plan_dev_cap = 0;
    Workspace ws;
    Stager stager;
    float* splitk_ws = nullptr;
    Workspace decode_ws;                   // of all decode steps over blocks that stay in place
    std::map<std::tuple<int, int, int>, std::unique_ptr<DecodeGraph>> graphs;
    int64_t decode_tick = 0;
    hipStream_t capture_stream = nullptr;
    const StepPlan* last_plan = nullptr;
    // timing by class of operation (PICOLM_ENGINE_TIME_OPS): an event before and after each one
    struct TimedOp {
        int cls;
        hipEvent_t before, after;
    };
    std::vector<TimedOp> timed;
    std::vector<hipEvent_t> spare_events;
    bool timing() const { return (flags & PICOLM_ENGINE_TIME_OPS) != 0; }
    // generation
    // (the sampled tokens of two steps in turn, [2][rows]: one is drawn while the other is still on its
    // way to the host; then the tokens picked for a smaller batch and their indices)
    int32_t* gen_tokens_dev = nullptr;     // [4][rows]: two draws, the picked tokens, the indices to pick
    int32_t* gen_tokens_host = nullptr;    // pinned, [2][rows]
    hipEvent_t gen_arrived[2] = {nullptr, nullptr};
    uint64_t* gen_states = nullptr;
    int32_t* gen_index = nullptr;
    void* gen_scratch = nullptr;
    size_t gen_scratch_bytes = 0;
    int gen_rows = 0;
    int prefill_step_tokens = 16384;       // most tokens of one prefill step of the generation loop
    bool host_only() const { return (flags & PICOLM_ENGINE_HOST_ONLY) != 0; }
};

static int dev_alloc(picolm_engine* e, void** p, size_t bytes, bool zero) {
    HIP_TRY(hipMalloc(p, std::max<size_t>(bytes, 256)));
    if (zero) HIP_TRY(hipMemset(*p, 0, std::max<size_t>(bytes, 256)));
    e->device_bytes += std::max<size_t>(bytes, 256);
    return 0;
}

// ---- creation ----------------------------------------------------------------------------------
static int check_program(const picolm_program* p, picolm_engine* e) {
    E_REQUIRE(-1, p && p->ops && p->n_ops > 0 && p->buffers && p->n_buffers > 0, "engine: an empty program");
    E_REQUIRE(-1, p->dtype == PICOLM_F32 || p->dtype == PICOLM_BF16, "engine: unknown dtype %d", p->dtype);
    E_REQUIRE(-1, p->vocab_size > 0, "engine: vocab_size %d", p->vocab_size);
    auto buf_ok = [&](int b) { return b >= 0 && b < p->n_buffers; };
    for (int i = 0; i < p->n_buffers; ++i) {
        const picolm_buffer& b = p->buffers[i];
        E_REQUIRE(-1, b.row_bytes > 0 && (b.rows == PICOLM_ROWS_STEP || b.rows == PICOLM_ROWS_WANTED) &&
                          (b.dtype == PICOLM_F32 || b.dtype == PICOLM_BF16),
                  "engine: buffer %d is ill-formed (row_bytes %d, rows %d, dtype %d)", i, b.row_bytes, b.rows, b.dtype);
    }
    E_REQUIRE(-1, buf_ok(p->logits_buffer) && p->buffers[p->logits_buffer].rows == PICOLM_ROWS_WANTED &&
                      p->buffers[p->logits_buffer].dtype == PICOLM_F32 &&
                      p->buffers[p->logits_buffer].row_bytes >= 4 * p->vocab_size,
              "engine: the logits buffer must hold float rows of the vocabulary's size for the wanted rows");
    for (int i = 0; i < p->n_ops; ++i) {
        const picolm_op& o = p->ops[i];
        E_REQUIRE(-1, o.rows == PICOLM_ROWS_STEP || o.rows == PICOLM_ROWS_WANTED, "engine: operation %d covers unknown rows %d", i, o.rows);
        E_REQUIRE(-1, buf_ok(o.out), "engine: operation %d writes buffer %d, there are %d", i, o.out, p->n_buffers);
        const picolm_buffer& out = p->buffers[o.out];
        switch (o.kind) {
            case PICOLM_OP_EMBED:
                E_REQUIRE(-1, o.weight && o.n == p->vocab_size && o.k > 0 && o.rows == PICOLM_ROWS_STEP,
                          "engine: operation %d (embedding) needs a table of vocab_size rows", i);
                E_REQUIRE(-1, out.dtype == PICOLM_F32 && out.row_bytes >= 4 * o.k && out.rows == PICOLM_ROWS_STEP,
                          "engine: operation %d (embedding) writes float rows of its width", i);
                break;
            case PICOLM_OP_RMSNORM: {
                E_REQUIRE(-1, buf_ok(o.in) && o.weight && o.k > 0 && o.eps > 0.f, "engine: operation %d (norm) is incomplete", i);
                const picolm_buffer& in = p->buffers[o.in];
                E_REQUIRE(-1, in.dtype == PICOLM_F32 && in.row_bytes >= 4 * o.k && in.rows == PICOLM_ROWS_STEP,
                          "engine: operation %d (norm) reads float rows of its width", i);
                E_REQUIRE(-1, out.row_bytes >= dt_bytes(out.dtype) * o.k && out.rows == o.rows,
                          "engine: operation %d (norm) writes rows of its width", i);
                break;
            }
            case PICOLM_OP_LINEAR: {
                E_REQUIRE(-1, buf_ok(o.in) && o.weight && o.n > 0 && o.k > 0 && o.epilogue >= 0 && o.epilogue <= 2,
                          "engine: operation %d (product) is incomplete", i);
                E_REQUIRE(-1, o.weight_dt == PICOLM_F32 || o.weight_dt == PICOLM_BF16, "engine: operation %d: weight dtype %d", i, o.weight_dt);
                const picolm_buffer& in = p->buffers[o.in];
                const int n_out = o.epilogue == 2 ? o.n / 2 : o.n;
                E_REQUIRE(-1, o.epilogue != 2 || o.n % 2 == 0, "engine: operation %d: the gated epilogue needs an even n", i);
                E_REQUIRE(-1, in.row_bytes >= dt_bytes(in.dtype) * o.k && in.rows == o.rows,
                          "engine: operation %d (product) reads rows of %d values", i, o.k);
                E_REQUIRE(-1, out.row_bytes >= dt_bytes(out.dtype) * n_out && out.rows == o.rows,
                          "engine: operation %d (product) writes rows of %d values", i, n_out);
                E_REQUIRE(-1, o.epilogue != 1 || out.dtype == PICOLM_F32, "engine: operation %d accumulates into float rows only", i);
                if (o.in_norm_weight) {
                    E_REQUIRE(-1, buf_ok(o.in_norm_x) && o.in_norm_eps > 0.f, "engine: operation %d: the norm of its input is incomplete", i);
                    const picolm_buffer& x = p->buffers[o.in_norm_x];
                    E_REQUIRE(-1, x.dtype == PICOLM_F32 && x.row_bytes >= 4 * o.k && x.rows == PICOLM_ROWS_STEP,
                              "engine: operation %d: the norm of its input reads float rows of %d values", i, o.k);
                }
                if (o.out_norm_weight) {
                    E_REQUIRE(-1, o.epilogue == 1 && o.out_norm_eps > 0.f, "engine: operation %d: only an accumulating product prepares a norm", i);
                    E_REQUIRE(-1, o.rows == PICOLM_ROWS_STEP, "engine: operation %d: only a product over every row of the step prepares a norm", i);
                    e->prep_n = std::max(e->prep_n, o.n);
                }
                break;
            }
            case PICOLM_OP_ATTENTION: {
                const int H = o.n_heads, G = o.n_kv_heads, d = o.head_dim;
                E_REQUIRE(-1, H > 0 && G > 0 && H % G == 0 && d >= 1 && d <= 1024, "engine: operation %d (attention): %d heads, %d groups, size %d", i, H, G, d);
                E_REQUIRE(-1, o.window >= 0, "engine: operation %d: a window of %d keys", i, o.window);
                E_REQUIRE(-1, buf_ok(o.in) && buf_ok(o.q_buffer) && o.rows == PICOLM_ROWS_STEP, "engine: operation %d (attention) is incomplete", i);
                const picolm_buffer &in = p->buffers[o.in], &q = p->buffers[o.q_buffer];
                E_REQUIRE(-1, in.dtype == PICOLM_F32 && in.row_bytes >= 4 * (H + 2 * G) * d, "engine: operation %d (attention) reads float rows of q, k, v", i);
                E_REQUIRE(-1, q.dtype == p->dtype && out.dtype == p->dtype && q.row_bytes >= dt_bytes(p->dtype) * H * d &&
                                  out.row_bytes >= dt_bytes(p->dtype) * H * d && out.rows == PICOLM_ROWS_STEP && q.rows == PICOLM_ROWS_STEP,
                          "engine: operation %d (attention) writes rows of %d values in the engine's dtype", i, H * d);
                E_REQUIRE(-1, o.kv_group >= 0 && o.kv_group < p->n_kv_groups, "engine: operation %d: cache group %d", i, o.kv_group);
                const picolm_kv_group& g = p->kv_groups[o.kv_group];
                E_REQUIRE(-1, o.kv_entry >= 0 && o.kv_entry < g.n_entries && g.n_kv_heads == G && g.head_dim == d && g.window == o.window,
                          "engine: operation %d does not fit its cache group", i);
                E_REQUIRE(-1, g.v_head_dim == 0 || g.v_head_dim == d,
                          "engine: operation %d: the attention operation takes keys and values of one size, its group has %d and %d", i, d,
                          g.v_head_dim);
                E_REQUIRE(-1, (o.cos_table == nullptr) == (o.sin_table == nullptr) && (o.rope_style == 0 || o.rope_style == 1) &&
                                  (!o.cos_table || d % 2 == 0),
                          "engine: operation %d: rotation needs both tables, a pairing of 0 or 1 and an even head size", i);
                E_REQUIRE(-1, o.scale > 0.f, "engine: operation %d: scale %g", i, o.scale);
                break;
            }
            case PICOLM_OP_CALL: {
                E_REQUIRE(-1, o.call != nullptr, "engine: operation %d (call) has no function", i);
                E_REQUIRE(-1, o.in == -1 || buf_ok(o.in), "engine: operation %d (call) reads buffer %d, there are %d", i, o.in, p->n_buffers);
                for (int x = 0; x < 4; ++x) {
                    E_REQUIRE(-1, o.extra[x] == -1 || buf_ok(o.extra[x]), "engine: operation %d (call) names buffer %d, there are %d", i,
                              o.extra[x], p->n_buffers);
                    E_REQUIRE(-1, o.extra[x] == -1 || p->buffers[o.extra[x]].rows == PICOLM_ROWS_STEP || o.rows == PICOLM_ROWS_WANTED,
                              "engine: operation %d (call) over every row names a buffer of the wanted rows", i);
                }
                E_REQUIRE(-1, out.rows == o.rows, "engine: operation %d (call) writes a buffer of other rows than it covers", i);
                E_REQUIRE(-1, o.in == -1 || p->buffers[o.in].rows == PICOLM_ROWS_STEP || o.rows == PICOLM_ROWS_WANTED,
                          "engine: operation %d (call) over every row reads a buffer of the wanted rows", i);
                if (o.call_flags & PICOLM_CALL_KV) {
                    E_REQUIRE(-1, o.kv_group >= 0 && o.kv_group < p->n_kv_groups && o.kv_entry >= 0 &&
                                      o.kv_entry < p->kv_groups[o.kv_group].n_entries && o.rows == PICOLM_ROWS_STEP,
                              "engine: operation %d (call): cache entry (%d, %d)", i, o.kv_group, o.kv_entry);
                } else {
                    E_REQUIRE(-1, !(o.call_flags & PICOLM_CALL_ATTENDS), "engine: operation %d (call) wants a work list without a cache entry", i);
                }
                if (o.call_flags & PICOLM_CALL_STATE)
                    E_REQUIRE(-1, o.state_group >= 0 && o.state_group < p->n_state_groups && o.state_entry >= 0 &&
                                      o.state_entry < p->state_groups[o.state_group].n_entries,
                              "engine: operation %d (call): state entry (%d, %d)", i, o.state_group, o.state_entry);
                E_REQUIRE(-1, o.tile_rows >= 0 && o.partial_floats >= 0, "engine: operation %d (call): tile_rows %d, partial_floats %d", i,
                          o.tile_rows, o.partial_floats);
                break;
            }
            default: E_REQUIRE(-1, false, "engine: operation %d has unknown kind %d", i, o.kind);
        }
    }
    return 0;
}

static void add_unique(std::vector<int>& v, int x) {
    if (std::find(v.begin(), v.end(), x) == v.end()) v.push_back(x);
}

static bool attn_on_matrix_cores(const picolm_engine* e, int H, int G, int d) {
    return e->dtype == PICOLM_BF16 && picolm_attn_mfma_fits(H, G, d);
}

extern "C" int picolm_engine_create(const picolm_program* program, int64_t max_tokens, int32_t max_seq_len, int32_t n_slots,
                                    int32_t flags, picolm_engine** out) {
    E_REQUIRE(-1, out != nullptr, "engine: no place for the handle");
    *out = nullptr;
    E_REQUIRE(PICOLM_ERR_CACHE, max_tokens > 0 && max_seq_len > 0, "the cache needs a positive token budget and sequence length");
    std::unique_ptr<picolm_engine> e(new picolm_engine);
    TRY(check_program(program, e.get()));
    e->flags = flags;
    e->dtype = program->dtype;
    e->vocab = program->vocab_size;
    e->ops.assign(program->ops, program->ops + program->n_ops);
    e->buffers.assign(program->buffers, program->buffers + program->n_buffers);
    e->logits_buffer = program->logits_buffer;
    if (!e->host_only()) TRY(picolm_device_check());
    const int n_pages = pages_for(max_tokens);
    e->max_seq_len = (int)std::min<int64_t>(max_seq_len, (int64_t)n_pages * PAGE_TOKENS);
    e->max_pages = pages_for(e->max_seq_len);
    e->n_slots = n_slots > 0 ? n_slots : n_pages;
    e->slots.init(e->n_slots);
    e->kv.resize(program->n_kv_groups);
    for (int gi = 0; gi < program->n_kv_groups; ++gi) {
        KVGroup& g = e->kv[gi];
        g.spec = program->kv_groups[gi];
        E_REQUIRE(-1, g.spec.n_entries > 0 && g.spec.n_kv_heads > 0 && g.spec.head_dim > 0 && g.spec.window >= 0 && g.spec.v_head_dim >= 0,
                  "engine: cache group %d is ill-formed", gi);
        g.max_pages = e->max_pages;
        // a window's ring: the window of the first query of a chunk of new tokens together with the
        // whole chunk, which is written before its queries are answered
        g.ring_pages = g.spec.window > 0 ? std::min(pages_for(g.spec.window - 1 + WINDOW_STEP_TOKENS) + 1, e->max_pages) : e->max_pages;
        g.n_pages = (int)std::min<int64_t>(n_pages, (int64_t)e->n_slots * g.ring_pages);
        g.pool.init(g.n_pages);
        g.pages.assign(e->n_slots, {});
        g.table_host.assign((size_t)e->n_slots * g.max_pages, 0);
        const size_t page_rows = (size_t)std::max(g.n_pages, 1) * g.spec.n_kv_heads * PAGE_TOKENS * dt_bytes(e->dtype);
        g.k_entry_bytes = page_rows * g.spec.head_dim;
        g.v_entry_bytes = page_rows * g.value_dim();
        if (!e->host_only()) {
            TRY(dev_alloc(e.get(), (void**)&g.k, g.k_entry_bytes * g.spec.n_entries, true));
            TRY(dev_alloc(e.get(), (void**)&g.v, g.v_entry_bytes * g.spec.n_entries, true));
            TRY(dev_alloc(e.get(), (void**)&g.table_dev, g.table_host.size() * 4, true));
        }
    }
    e->state.resize(program->n_state_groups);
    for (int gi = 0; gi < program->n_state_groups; ++gi) {
        StateGroup& s = e->state[gi];
        s.spec = program->state_groups[gi];
        E_REQUIRE(-1, s.spec.n_entries > 0 && s.spec.bytes_per_slot > 0, "engine: state group %d is ill-formed", gi);
        if (!e->host_only())
            TRY(dev_alloc(e.get(), (void**)&s.data, (size_t)s.spec.n_entries * e->n_slots * s.spec.bytes_per_slot, true));
    }
    e->group_written.assign(e->kv.size(), 0);
    e->group_attended.assign(e->kv.size(), 0);
    e->recordable = true;
    for (const picolm_op& o : e->ops) {
        if (o.kind == PICOLM_OP_CALL) {
            if (!(o.call_flags & PICOLM_CALL_RECORDABLE)) e->recordable = false;
            if (!(o.call_flags & PICOLM_CALL_KV)) continue;
            const KVGroup& g = e->kv[o.kv_group];
            if (g.is_ring()) e->call_on_ring = true;
            if (o.kv_writes) e->group_written[o.kv_group] = 1;
            if (!(o.call_flags & PICOLM_CALL_ATTENDS)) continue;
            e->group_attended[o.kv_group] = 1;
            if (o.tile_rows > 0) add_unique(e->tile_rows, o.tile_rows);
            e->decode_blocks_per_chunk = std::max(e->decode_blocks_per_chunk, g.spec.n_kv_heads);
            e->decode_max_pages_per_chunk = std::min(e->decode_max_pages_per_chunk, 16);
            e->counters_needed = std::max(e->counters_needed, e->n_slots * g.spec.n_kv_heads * 4);
            e->partial_floats_per_seq_chunk = std::max(e->partial_floats_per_seq_chunk, (size_t)o.partial_floats);
            continue;
        }
        if (o.kind != PICOLM_OP_ATTENTION) continue;
        E_REQUIRE(-1, !o.cos_table || o.table_positions >= e->max_seq_len,
                  "engine: rotation tables for %d positions, the cache takes sequences of %d", o.table_positions, e->max_seq_len);
        if (o.kv_writes) e->group_written[o.kv_group] = 1;
        e->group_attended[o.kv_group] = 1;
        const int R = o.n_heads / o.n_kv_heads;
        const bool mfma = !e->host_only() && attn_on_matrix_cores(e.get(), o.n_heads, o.n_kv_heads, o.head_dim);
        add_unique(e->tile_rows, mfma ? picolm_attn_prefill_mfma_tile_tokens(o.n_heads, o.n_kv_heads) : picolm_attn_prefill_tile_rows());
        // workgroups a chunk of the decode work list gets: the widest launch sizes the step's list
        e->decode_blocks_per_chunk = std::max(e->decode_blocks_per_chunk, o.n_kv_heads * ((R + (mfma ? 31 : 15)) / (mfma ? 32 : 16)));
        e->decode_max_pages_per_chunk = std::min(e->decode_max_pages_per_chunk, mfma ? 64 : 16);
        e->counters_needed = std::max(e->counters_needed, e->n_slots * o.n_kv_heads * ((R + 31) / 32));
        e->partial_floats_per_seq_chunk = std::max(e->partial_floats_per_seq_chunk, (size_t)o.n_heads * (o.head_dim + 2));
    }
    if (!e->host_only()) {
        TRY(dev_alloc(e.get(), (void**)&e->splitk_ws, (size_t)picolm_linear_workspace_floats() * 4, false));
        HIP_TRY(hipStreamCreateWithFlags(&e->capture_stream, hipStreamNonBlocking));
    }
    *out = e.release();
    return 0;
}

static void free_workspace(Workspace& w) {
    if (w.base) (void)hipFree(w.base);
    if (w.counters) (void)hipFree(w.counters);
    w.base = nullptr;
    w.counters = nullptr;
}

static void free_decode_graph(picolm_engine* e, DecodeGraph& g) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (g.batch.dev) {
        (void)hipFree(g.batch.dev);
        e->device_bytes -= g.batch.plan.ints.size() * 4;
    }
    for (int t = 0; t < 2; ++t) {
        if (g.batch.pinned[t]) (void)hipHostFree(g.batch.pinned[t]);
        if (g.batch.sent[t]) (void)hipEventDestroy(g.batch.sent[t]);
    }
}

extern "C" void picolm_engine_destroy(picolm_engine* e) {
    if (!e) return;
    if (!e->host_only()) (void)hipDeviceSynchronize();
    for (auto& kvp : e->graphs) free_decode_graph(e, *kvp.second);
    free_workspace(e->decode_ws);
    for (KVGroup& g : e->kv) {
        if (g.k) (void)hipFree(g.k);
        if (g.v) (void)hipFree(g.v);
        if (g.table_dev) (void)hipFree(g.table_dev);
    }
    for (StateGroup& s : e->state)
        if (s.data) (void)hipFree(s.data);
    free_workspace(e->ws);
    if (e->plan_dev) (void)hipFree(e->plan_dev);
    if (e->splitk_ws) (void)hipFree(e->splitk_ws);
    if (e->gen_tokens_dev) (void)hipFree(e->gen_tokens_dev);
    if (e->gen_tokens_host) (void)hipHostFree(e->gen_tokens_host);
    if (e->gen_states) (void)hipFree(e->gen_states);
    if (e->gen_index) (void)hipFree(e->gen_index);
    if (e->gen_scratch) (void)hipFree(e->gen_scratch);
    for (int t = 0; t < 2; ++t)
        if (e->gen_arrived[t]) (void)hipEventDestroy(e->gen_arrived[t]);
    e->stager.destroy();
    for (auto& t : e->timed) {
        (void)hipEventDestroy(t.before);
        (void)hipEventDestroy(t.after);
    }
    for (auto ev : e->spare_events) (void)hipEventDestroy(ev);
    if (e->capture_stream) (void)hipStreamDestroy(e->capture_stream);
    delete e;
}

// ---- slots and pages ---------------------------------------------------------------------------
extern "C" int picolm_engine_slot_alloc(picolm_engine* e, int32_t* slot, hipStream_t stream) {
    E_REQUIRE(-1, e && slot, "slot_alloc: null argument");
    E_REQUIRE(PICOLM_ERR_CACHE_FULL, !e->slots.free_.empty(), "all %d slots are live", e->n_slots);
    const int s = e->slots.free_.back();
    e->slots.free_.pop_back();
    e->slots.live[s] = 1;
    e->slots.length[s] = 0;
    e->version++;
    if (!e->host_only())        // (outside any recorded step: steps are recorded on a stream of the engine's own)
        for (StateGroup& g : e->state)
            for (int en = 0; en < g.spec.n_entries; ++en)
                HIP_TRY(hipMemsetAsync(g.data + ((size_t)en * e->n_slots + s) * g.spec.bytes_per_slot, 0, g.spec.bytes_per_slot, stream));
    *slot = s;
    return 0;
}

extern "C" int picolm_engine_slot_free(picolm_engine* e, int32_t slot) {
    E_REQUIRE(-1, e, "slot_free: null engine");
    E_REQUIRE(PICOLM_ERR_CACHE, slot >= 0 && slot < e->n_slots, "slot %d does not exist", slot);
    E_REQUIRE(PICOLM_ERR_CACHE, e->slots.live[slot], "slot %d is freed twice", slot);
    e->slots.live[slot] = 0;
    e->slots.length[slot] = 0;
    e->slots.free_.push_back(slot);
    e->version++;
    for (KVGroup& g : e->kv) {
        g.pool.give(g.pages[slot]);
        g.pages[slot].clear();
    }
    return 0;
}

extern "C" int picolm_engine_slot_length(picolm_engine* e, int32_t slot) {
    if (!e || !e->slots.is_live(slot)) return -1;
    return e->slots.length[slot];
}

// Pages for lengths[i] tokens in slots[i], in every group: all or nothing.
static int reserve_many(picolm_engine* e, const std::vector<int>& slots, const std::vector<int>& lengths) {
    for (size_t i = 0; i < slots.size(); ++i) {
        E_REQUIRE(PICOLM_ERR_CACHE, e->slots.is_live(slots[i]), "slot %d is not live", slots[i]);
        E_REQUIRE(PICOLM_ERR_CACHE_FULL, lengths[i] <= e->max_seq_len, "a sequence of %d tokens exceeds the cache's %d", lengths[i],
                  e->max_seq_len);
    }
    for (KVGroup& g : e->kv) {
        int64_t need = 0;
        for (size_t i = 0; i < slots.size(); ++i) need += g.missing(slots[i], lengths[i]);
        E_REQUIRE(PICOLM_ERR_CACHE_FULL, need <= g.pool.n_free(), "the batch needs %lld more pages, %d are free", (long long)need,
                  g.pool.n_free());
    }
    for (KVGroup& g : e->kv)
        for (size_t i = 0; i < slots.size(); ++i) {
            const int s = slots[i], k = g.missing(s, lengths[i]);
            if (k == 0) continue;
            const int first = (int)g.pages[s].size();
            g.pool.take(k, g.pages[s]);
            for (int j = first; j < first + k; ++j) g.table_host[(size_t)s * g.max_pages + j] = g.pages[s][j];
            add_unique(g.dirty, s);
            e->version += k;
        }
    return 0;
}

// Bring the device page tables up to date (rows of slots that got pages).
static int flush_tables(picolm_engine* e, hipStream_t stream) {
    for (KVGroup& g : e->kv) {
        if (!e->host_only())
            for (int s : g.dirty)
                TRY(e->stager.upload(g.table_dev + (size_t)s * g.max_pages, &g.table_host[(size_t)s * g.max_pages],
                                     (size_t)g.max_pages * 4, stream));
        g.dirty.clear();
    }
    return 0;
}

// ---- planning a step ---------------------------------------------------------------------------
static Span put(StepPlan& p, const std::vector<int32_t>& v) {
    Span s;
    s.n = (int)v.size();
    s.off = p.take(std::max(s.n, 1));
    std::copy(v.begin(), v.end(), p.ints.begin() + s.off);
    return s;
}

static void plan_write_pages(picolm_engine* e, StepPlan& p, const std::vector<int32_t>& tok_seq, const std::vector<int32_t>& tok_pos) {
    p.write_pages.assign(e->kv.size(), Span{});
    for (size_t gi = 0; gi < e->kv.size(); ++gi) {
        if (!e->group_written[gi]) continue;
        const KVGroup& g = e->kv[gi];
        std::vector<int32_t> pages(p.T);
        for (int t = 0; t < p.T; ++t)
            pages[t] = g.table_host[(size_t)p.slots[tok_seq[t]] * g.max_pages + (tok_pos[t] / PAGE_TOKENS) % g.ring_pages];
        p.write_pages[gi] = put(p, pages);
    }
}

// The tiles of `rpt` new tokens of a prefill step (or of a slice of one), sorted by the keys a tile
// sees: the kernels hand out the longest first.
static TileList plan_tiles(StepPlan& p, const std::vector<int>& pos0, const std::vector<int>& n_new, int rpt) {
    struct Tile {
        int keys, seq, q0;
    };
    std::vector<Tile> tiles;
    for (int i = 0; i < (int)n_new.size(); ++i)
        for (int q0 = 0; q0 < n_new[i]; q0 += rpt) tiles.push_back({pos0[i] + std::min(q0 + rpt, n_new[i]), i, q0});
    std::sort(tiles.begin(), tiles.end(), [](const Tile& a, const Tile& b) {
        return a.keys != b.keys ? a.keys < b.keys : a.seq != b.seq ? a.seq < b.seq : a.q0 < b.q0;
    });
    std::vector<int32_t> seqs, q0s;
    for (auto& t : tiles) {
        seqs.push_back(t.seq);
        q0s.push_back(t.q0);
    }
    TileList tl;
    tl.rows_per_tile = rpt;
    tl.n = (int)tiles.size();
    tl.seq = put(p, seqs);
    tl.q0 = put(p, q0s);
    return tl;
}

// Builds the index arrays of a step that is not a recorded decode step.  The sequences and their
// tokens have been checked, and the pages reserved.
static void plan_step(picolm_engine* e, StepPlan& p, const std::vector<int>& slots, const std::vector<int>& pos0,
                      const std::vector<int>& n_new, const int32_t* tokens, const std::vector<std::vector<int>>& want) {
    p = StepPlan();
    p.n_seq = (int)slots.size();
    p.slots = slots;
    p.pos0 = pos0;
    p.n_new = n_new;
    std::vector<int32_t> cu(p.n_seq + 1, 0), tok_pos, tok_seq, rows;
    for (int i = 0; i < p.n_seq; ++i) {
        cu[i + 1] = cu[i] + n_new[i];
        p.max_new = std::max(p.max_new, n_new[i]);
        for (int j = 0; j < n_new[i]; ++j) {
            tok_pos.push_back(pos0[i] + j);
            tok_seq.push_back(i);
        }
        for (int j : want[i]) rows.push_back(cu[i] + j);
    }
    p.T = cu[p.n_seq];
    p.is_decode = p.max_new == 1;
    p.n_want = (int)rows.size();
    p.every_row = p.n_want == p.T;
    for (int r = 0; p.every_row && r < p.T; ++r) p.every_row = rows[r] == r;
    p.seq_slot = put(p, std::vector<int32_t>(slots.begin(), slots.end()));
    p.seq_pos0 = put(p, std::vector<int32_t>(pos0.begin(), pos0.end()));
    p.seq_nnew = put(p, std::vector<int32_t>(n_new.begin(), n_new.end()));
    p.cu_seqlens = put(p, cu);
    p.tok_pos = put(p, tok_pos);
    p.tok_seq = put(p, tok_seq);
    p.tokens = put(p, std::vector<int32_t>(tokens, tokens + p.T));
    p.want_rows = put(p, rows);
    plan_write_pages(e, p, tok_seq, tok_pos);
    p.lists.assign(e->kv.size(), DecodeList{});
    if (p.is_decode) {
        p.pages_per_chunk = decode_pages_per_chunk(pos0, e->decode_blocks_per_chunk, e->decode_max_pages_per_chunk);
        for (size_t gi = 0; gi < e->kv.size(); ++gi) {
            if (!e->group_attended[gi]) continue;
            int n = 0;
            for (int q : pos0) n += chunks_of(e->kv[gi], q, p.pages_per_chunk);
            DecodeList& l = p.lists[gi];
            l.span.n = 8 * (n + 1);
            l.span.off = p.take(l.span.n);
            l.n_chunks = fill_chunk_list(&p.ints[l.span.off], slots, pos0, p.pages_per_chunk, e->kv[gi], &l.most);
        }
    } else {
        for (int rpt : e->tile_rows) p.tiles.push_back(plan_tiles(p, pos0, n_new, rpt));
        bool rings = false;
        for (size_t gi = 0; gi < e->kv.size(); ++gi) rings = rings || (e->group_attended[gi] && e->kv[gi].is_ring());
        if (rings && p.max_new > WINDOW_STEP_TOKENS) {
            // the step cut along positions: chunk c holds, of every sequence that has them, its new
            // tokens c * 256 .. c * 256 + 255
            for (int lo = 0; lo < p.max_new; lo += WINDOW_STEP_TOKENS) {
                WindowChunk c;
                std::vector<int32_t> sl, ps, nn, first, rows;
                std::vector<int> cpos, cnew;
                for (int i = 0; i < p.n_seq; ++i) {
                    if (n_new[i] <= lo) continue;
                    const int n = std::min(WINDOW_STEP_TOKENS, n_new[i] - lo);
                    sl.push_back(slots[i]);
                    ps.push_back(pos0[i] + lo);
                    nn.push_back(n);
                    first.push_back(cu[i] + lo);
                    cpos.push_back(pos0[i] + lo);
                    cnew.push_back(n);
                    for (int j = 0; j < n; ++j) rows.push_back(cu[i] + lo + j);
                }
                c.n_seq = (int)sl.size();
                c.n_rows = (int)rows.size();
                c.seq_slot = put(p, sl);
                c.seq_pos0 = put(p, ps);
                c.seq_nnew = put(p, nn);
                c.first_row = put(p, first);
                c.rows = put(p, rows);
                for (int rpt : e->tile_rows) c.tiles.push_back(plan_tiles(p, cpos, cnew, rpt));
                p.window_chunks.push_back(c);
            }
        }
    }
}

static int upload_plan(picolm_engine* e, StepPlan& p, hipStream_t stream) {
    if (e->host_only()) return 0;
    const size_t bytes = p.ints.size() * 4;
    if (bytes > e->plan_dev_cap) {
        if (e->plan_dev) {
            HIP_TRY(hipStreamSynchronize(stream));      // kernels of an earlier step may still read the old block
            HIP_TRY(hipFree(e->plan_dev));
            e->device_bytes -= e->plan_dev_cap;
        }
        e->plan_dev_cap = align_up(bytes * 2, 4096);
        HIP_TRY(hipMalloc((void**)&e->plan_dev, e->plan_dev_cap));
        e->device_bytes += e->plan_dev_cap;
    }
    p.dev = e->plan_dev;
    return e->stager.upload(e->plan_dev, p.ints.data(), bytes, stream);
}

// ---- recorded decode steps: the block that stays in place --------------------------------------
static int decode_batch_init(picolm_engine* e, DecodeBatch& b, int n_seq, int ppc, int most_chunks) {
    StepPlan& p = b.plan;
    p = StepPlan();
    p.n_seq = p.T = p.n_want = n_seq;
    p.max_new = 1;
    p.is_decode = p.every_row = true;
    p.pages_per_chunk = ppc;
    p.n_new.assign(n_seq, 1);
    std::vector<int32_t> zeros(n_seq, 0), ones(n_seq, 1), ar(n_seq + 1);
    for (int i = 0; i <= n_seq; ++i) ar[i] = i;
    p.seq_slot = put(p, zeros);
    p.seq_pos0 = put(p, zeros);
    p.seq_nnew = put(p, ones);
    p.cu_seqlens = put(p, ar);
    p.tok_pos = put(p, zeros);
    p.tok_seq = put(p, std::vector<int32_t>(ar.begin(), ar.begin() + n_seq));
    p.tokens = put(p, zeros);
    p.want_rows = put(p, std::vector<int32_t>(ar.begin(), ar.begin() + n_seq));
    p.write_pages.assign(e->kv.size(), Span{});
    p.lists.assign(e->kv.size(), DecodeList{});
    b.live.assign(e->kv.size(), 0);
    for (size_t gi = 0; gi < e->kv.size(); ++gi) {
        if (e->group_written[gi]) p.write_pages[gi] = put(p, zeros);
        if (e->group_attended[gi]) {
            // a list of fixed capacity: every sequence with `most_chunks` chunks (or as many as the
            // group's pages make); entries not in use hold what an earlier step left, and the
            // header says how many are
            DecodeList& l = p.lists[gi];
            l.most = std::min(most_chunks, (e->kv[gi].ring_pages + ppc - 1) / ppc);
            l.n_chunks = n_seq * l.most;
            l.span.n = 8 * (l.n_chunks + 1);
            l.span.off = p.take(l.span.n);
        }
    }
    if (e->host_only()) return 0;
    const size_t bytes = p.ints.size() * 4;
    HIP_TRY(hipMalloc((void**)&b.dev, bytes));
    HIP_TRY(hipMemset(b.dev, 0, bytes));
    e->device_bytes += bytes;
    p.dev = b.dev;
    for (int t = 0; t < 2; ++t) {
        HIP_TRY(hipHostMalloc((void**)&b.pinned[t], bytes, hipHostMallocDefault));
        HIP_TRY(hipEventCreateWithFlags(&b.sent[t], hipEventDisableTiming));
    }
    return 0;
}

// `tokens` null: they are on the device and are copied into the block by the caller.
static int decode_batch_fill(picolm_engine* e, DecodeBatch& b, const std::vector<int>& slots, const std::vector<int>& pos0,
                             const int32_t* tokens, hipStream_t stream) {
    StepPlan& p = b.plan;
    const int n = p.n_seq;
    // between page boundaries only the positions move: the lists and pages stay as they are,
    // as long as no slot or page of the cache has changed hands
    bool same_pages = b.filled && b.cache_version == e->version && slots == p.slots;
    for (int i = 0; same_pages && i < n; ++i) same_pages = pos0[i] == p.pos0[i] + 1 && pos0[i] % PAGE_TOKENS != 0;
    b.cache_version = e->version;
    b.filled = true;
    p.slots = slots;
    p.pos0 = pos0;
    for (int i = 0; i < n; ++i) {
        p.ints[p.seq_slot.off + i] = slots[i];
        p.ints[p.seq_pos0.off + i] = pos0[i];
        p.ints[p.tok_pos.off + i] = pos0[i];
        if (tokens) p.ints[p.tokens.off + i] = tokens[i];
    }
    for (size_t gi = 0; gi < e->kv.size(); ++gi) {
        const KVGroup& g = e->kv[gi];
        DecodeList& l = p.lists[gi];
        if (l.span.n) {
            int32_t* list = &p.ints[l.span.off];
            if (same_pages && g.spec.window == 0) {        // (a window's first page can move on any step)
                for (int x = 0; x < b.live[gi]; ++x) list[8 * (x + 1) + 2] += 1;
            } else {
                int chunks = 0;
                for (int q : pos0) {
                    E_REQUIRE(PICOLM_ERR_STEP, chunks_of(g, q, p.pages_per_chunk) <= l.most,
                              "a decode step's work list was laid out for %d chunks a sequence, one needs %d", l.most,
                              chunks_of(g, q, p.pages_per_chunk));
                    chunks += chunks_of(g, q, p.pages_per_chunk);
                }
                E_REQUIRE(PICOLM_ERR_STEP, chunks <= l.n_chunks, "a decode step's work list holds %d chunks, %d are needed", l.n_chunks, chunks);
                int most = 0;
                b.live[gi] = fill_chunk_list(list, slots, pos0, p.pages_per_chunk, g, &most);
            }
        }
        if (p.write_pages[gi].n && !same_pages)
            for (int i = 0; i < n; ++i)
                p.ints[p.write_pages[gi].off + i] = g.table_host[(size_t)slots[i] * g.max_pages + (pos0[i] / PAGE_TOKENS) % g.ring_pages];
    }
    if (e->host_only()) return 0;
    // through one of two pinned copies, in turn; a copy is written again only after the transfer
    // that read it has ended
    const int t = b.turn;
    b.turn ^= 1;
    if (b.sent_once[t]) HIP_TRY(hipEventSynchronize(b.sent[t]));
    const size_t bytes = p.ints.size() * 4;
    memcpy(b.pinned[t], p.ints.data(), bytes);
    HIP_TRY(hipMemcpyAsync(b.dev, b.pinned[t], bytes, hipMemcpyHostToDevice, stream));
    HIP_TRY(hipEventRecord(b.sent[t], stream));
    b.sent_once[t] = true;
    return 0;
}

// ---- workspace -------------------------------------------------------------------------------
static int workspace_ensure(picolm_engine* e, Workspace& w, const StepPlan& p, int most) {
    if (!w.counters && e->counters_needed) TRY(dev_alloc(e, (void**)&w.counters, (size_t)e->counters_needed * 4, true));
    if (w.for_T == p.T && w.for_want == p.n_want && w.for_seq == p.n_seq && w.for_most == most && w.base) return 0;
    size_t off = 0;
    w.offsets.resize(e->buffers.size());
    for (size_t i = 0; i < e->buffers.size(); ++i) {
        w.offsets[i] = off;
        const int rows = e->buffers[i].rows == PICOLM_ROWS_STEP ? p.T : p.n_want;
        off = align_up(off + (size_t)std::max(rows, 1) * e->buffers[i].row_bytes, 256);
    }
    if (e->prep_n) {
        int parts = 0;
        for (const picolm_op& o : e->ops)
            if (o.kind == PICOLM_OP_LINEAR && o.out_norm_weight) parts = std::max(parts, picolm_linear_norm_parts(p.T, o.n, o.k));
        for (int f = 0; f < 2; ++f) {
            w.prep_h[f] = off;
            off = align_up(off + (size_t)p.T * e->prep_n * 2, 256);
            w.prep_ssq[f] = off;
            off = align_up(off + (size_t)std::max(parts, 1) * picolm_linear_norm_rows(p.T) * 4, 256);
        }
    }
    w.partial = off;
    if (p.is_decode && most > 1) off = align_up(off + (size_t)p.n_seq * most * e->partial_floats_per_seq_chunk * 4, 256);
    if (off > w.cap) {
        if (w.base) {
            HIP_TRY(hipDeviceSynchronize());        // an earlier step's kernels may still use the old memory
            HIP_TRY(hipFree(w.base));
            e->device_bytes -= w.cap;
            w.base = nullptr;
        }
        w.cap = align_up(off + off / 8, 1 << 16);
        HIP_TRY(hipMalloc((void**)&w.base, w.cap));
        e->device_bytes += w.cap;
        w.generation++;
    }
    w.for_T = p.T;
    w.for_want = p.n_want;
    w.for_seq = p.n_seq;
    w.for_most = most;
    return 0;
}

// ---- the operations ------------------------------------------------------------------------------
struct Run {
    picolm_engine* e;
    const StepPlan& p;
    Workspace& w;
    hipStream_t stream;
    Prepared prepared;
    char* buf(int b) const { return w.base + w.offsets[b]; }
};

static int run_linear(Run& r, const picolm_op& o) {
    picolm_engine* e = r.e;
    const StepPlan& p = r.p;
    const int M = o.rows == PICOLM_ROWS_STEP ? p.T : p.n_want;
    const picolm_buffer &bi = e->buffers[o.in], &bo = e->buffers[o.out];
    const void* a = r.buf(o.in);
    int a_dt = bi.dtype;
    void* c = r.buf(o.out);
    const float* ssq = nullptr;
    int n_parts = 0, norm_len = 0;
    float eps = 0.f;
    if (o.in_norm_weight) {
        // whoever applies a norm next takes what the product before prepared for it, or nothing
        const Prepared got = r.prepared;
        r.prepared = Prepared();
        const char* x = r.buf(o.in_norm_x);
        const bool all_rows = o.rows == PICOLM_ROWS_STEP || p.every_row;
        if (got.x == x && got.w == o.in_norm_weight && got.eps == o.in_norm_eps && all_rows &&
            picolm_linear_links_norms(got.h, PICOLM_BF16, o.weight, o.weight_dt, bo.dtype, M, o.n, o.k, o.epilogue, 0)) {
            a = got.h;
            a_dt = PICOLM_BF16;
            ssq = got.ssq;
            n_parts = got.parts;
            norm_len = o.k;
            eps = o.in_norm_eps;
        } else {
            TRY(picolm_rmsnorm((const float*)x, o.in_norm_weight, r.buf(o.in), bi.dtype, all_rows ? nullptr : p.at(p.want_rows), M,
                               o.k, o.in_norm_eps, r.stream));
        }
    }
    const float* next_w = nullptr;
    void* next_h = nullptr;
    float* next_ssq = nullptr;
    int next_parts = 0;
    if (o.out_norm_weight && o.epilogue == 1 && (o.out_norm_when == 0 || (p.every_row && p.n_want > 0)) &&
        picolm_linear_links_norms(a, a_dt, o.weight, o.weight_dt, bo.dtype, M, o.n, o.k, o.epilogue, 1)) {
        r.w.flip ^= 1;
        next_w = o.out_norm_weight;
        next_h = r.w.base + r.w.prep_h[r.w.flip];
        next_ssq = (float*)(r.w.base + r.w.prep_ssq[r.w.flip]);
        next_parts = picolm_linear_norm_parts(M, o.n, o.k);
    }
    TRY(picolm_linear(a, a_dt, o.weight, o.weight_dt, c, bo.dtype, M, o.n, o.k, o.epilogue, next_w, next_h, next_ssq, next_parts, ssq,
                      n_parts, norm_len, eps, e->splitk_ws, r.stream));
    if (next_w) {
        r.prepared.by = &o;
        r.prepared.x = c;
        r.prepared.w = o.out_norm_weight;
        r.prepared.eps = o.out_norm_eps;
        r.prepared.h = next_h;
        r.prepared.ssq = next_ssq;
        r.prepared.parts = next_parts;
    }
    return 0;
}

// picolm's order (picolm/model_core.c:1849-2151): rotate q and k, write k and v to the cache,
// attend over keys t <= pos.
static int run_attention(Run& r, const picolm_op& o) {
    picolm_engine* e = r.e;
    const StepPlan& p = r.p;
    const KVGroup& g = e->kv[o.kv_group];
    const int H = o.n_heads, G = o.n_kv_heads, d = o.head_dim, dt = e->dtype;
    const float* qkv = (const float*)r.buf(o.in);
    void* q = r.buf(o.q_buffer);
    void* out = r.buf(o.out);
    char* k_pages = g.k + (size_t)o.kv_entry * g.k_entry_bytes;
    char* v_pages = g.v + (size_t)o.kv_entry * g.v_entry_bytes;
    const bool writes = o.kv_writes != 0;
    const int32_t* tok_page = writes ? p.at(p.write_pages[o.kv_group]) : nullptr;
    const bool mfma = attn_on_matrix_cores(e, H, G, d);
    if (p.is_decode) {
        const DecodeList& l = p.lists[o.kv_group];
        float* partial = l.most > 1 ? (float*)(r.w.base + r.w.partial) : nullptr;
        int32_t* done = l.most > 1 ? r.w.counters : nullptr;
        if (writes && mfma)         // rotation, cache write and attention in one launch
            return picolm_attn_decode_rope_mfma(qkv, k_pages, v_pages, out, partial, p.n_seq, p.at(l.span), l.n_chunks, p.pages_per_chunk,
                                                l.most, p.at(p.seq_pos0), g.table_dev, g.max_pages, g.ring_pages, H, G, d, o.window,
                                                o.scale, o.cos_table, o.sin_table, o.rope_style, tok_page, done, r.stream);
        TRY(picolm_rope_kv_store(qkv, q, writes ? k_pages : nullptr, writes ? v_pages : nullptr, dt, o.cos_table, o.sin_table, o.rope_style,
                                 p.at(p.tok_pos), tok_page, p.T, H, G, d, nullptr, r.stream));
        if (mfma)
            return picolm_attn_decode_mfma(q, k_pages, v_pages, out, partial, p.n_seq, p.at(l.span), l.n_chunks, p.pages_per_chunk, l.most,
                                           p.at(p.seq_pos0), g.table_dev, g.max_pages, g.ring_pages, H, G, d, o.window, o.scale, done,
                                           r.stream);
        return picolm_attn_decode_generic(q, k_pages, v_pages, out, partial, dt, p.n_seq, p.at(l.span), l.n_chunks, p.pages_per_chunk,
                                          l.most, p.at(p.seq_pos0), g.table_dev, g.max_pages, g.ring_pages, H, G, d, o.window, o.scale,
                                          r.stream);
    }
    const int tile_rows = mfma ? picolm_attn_prefill_mfma_tile_tokens(H, G) : picolm_attn_prefill_tile_rows();
    if (g.is_ring() && !p.window_chunks.empty()) {
        // a ring holds a window and one chunk of new tokens: write and answer the step chunk by chunk
        for (const WindowChunk& c : p.window_chunks) {
            const TileList* ct = c.tiles_of(tile_rows);
            E_REQUIRE(-1, ct != nullptr, "attention: the step has no tiles of the height this kernel takes");
            TRY(picolm_rope_kv_store(qkv, q, writes ? k_pages : nullptr, writes ? v_pages : nullptr, dt, o.cos_table, o.sin_table,
                                     o.rope_style, p.at(p.tok_pos), tok_page, c.n_rows, H, G, d, p.at(c.rows), r.stream));
            if (mfma)
                TRY(picolm_attn_prefill_mfma(q, k_pages, v_pages, out, p.at(ct->seq), p.at(ct->q0), ct->n, p.at(c.seq_slot), p.at(c.seq_pos0),
                                             p.at(c.seq_nnew), p.at(c.first_row), g.table_dev, g.max_pages, g.ring_pages, H, G, d, o.window,
                                             o.scale, r.stream));
            else
                TRY(picolm_attn_prefill_generic(q, k_pages, v_pages, out, dt, p.at(ct->seq), p.at(ct->q0), ct->n, p.at(c.seq_slot),
                                                p.at(c.seq_pos0), p.at(c.seq_nnew), p.at(c.first_row), g.table_dev, g.max_pages,
                                                g.ring_pages, H, G, d, o.window, o.scale, r.stream));
        }
        return 0;
    }
    const TileList* tl = p.tiles_of(tile_rows);
    E_REQUIRE(-1, tl != nullptr, "attention: the step has no tiles of the height this kernel takes");
    if (mfma && picolm_attn_prefill_rotates_q(p.T)) {      // keys and values go to the cache; the attention kernel rotates q on its way in
        if (writes)
            TRY(picolm_kv_store_tiles(qkv, k_pages, v_pages, dt, o.cos_table, o.sin_table, o.rope_style, p.at(tl->seq), p.at(tl->q0), tl->n,
                                      tl->rows_per_tile, p.at(p.seq_slot), p.at(p.seq_pos0), p.at(p.seq_nnew), p.at(p.cu_seqlens),
                                      g.table_dev, g.max_pages, g.ring_pages, H, G, d, r.stream));
        return picolm_attn_prefill_rope_mfma(qkv, k_pages, v_pages, out, p.at(tl->seq), p.at(tl->q0), tl->n, p.at(p.seq_slot),
                                             p.at(p.seq_pos0), p.at(p.seq_nnew), p.at(p.cu_seqlens), g.table_dev, g.max_pages,
                                             g.ring_pages, H, G, d, o.window, o.scale, o.cos_table, o.sin_table, o.rope_style, r.stream);
    }
    TRY(picolm_rope_kv_store(qkv, q, writes ? k_pages : nullptr, writes ? v_pages : nullptr, dt, o.cos_table, o.sin_table, o.rope_style,
                             p.at(p.tok_pos), tok_page, p.T, H, G, d, nullptr, r.stream));
    if (mfma)
        return picolm_attn_prefill_mfma(q, k_pages, v_pages, out, p.at(tl->seq), p.at(tl->q0), tl->n, p.at(p.seq_slot), p.at(p.seq_pos0),
                                        p.at(p.seq_nnew), p.at(p.cu_seqlens), g.table_dev, g.max_pages, g.ring_pages, H, G, d, o.window,
                                        o.scale, r.stream);
    return picolm_attn_prefill_generic(q, k_pages, v_pages, out, dt, p.at(tl->seq), p.at(tl->q0), tl->n, p.at(p.seq_slot),
                                       p.at(p.seq_pos0), p.at(p.seq_nnew), p.at(p.cu_seqlens), g.table_dev, g.max_pages, g.ring_pages, H,
                                       G, d, o.window, o.scale, r.stream);
}

// An operation of the caller's: it is handed what the engine knows of the step and queues its own
// work on the step's stream (picolm's layer loop branches per layer kind in C instead,
// picolm/model_core.c:1824-1839).
static int run_call(Run& r, const picolm_op& o) {
    picolm_engine* e = r.e;
    const StepPlan& p = r.p;
    picolm_step_view v;
    memset(&v, 0, sizeof(v));
    v.struct_bytes = (int32_t)sizeof(v);
    v.dtype = e->dtype;
    v.n_seq = p.n_seq;
    v.n_tokens = p.T;
    v.n_wanted = p.n_want;
    v.is_decode = p.is_decode;
    v.every_row_wanted = p.every_row;
    v.recording = r.stream == e->capture_stream && e->capture_stream != nullptr;
    v.slots = p.slots.data();
    v.pos0 = p.pos0.data();
    v.n_new = p.n_new.data();
    v.seq_slot = p.at(p.seq_slot);
    v.seq_pos0 = p.at(p.seq_pos0);
    v.seq_nnew = p.at(p.seq_nnew);
    v.cu_seqlens = p.at(p.cu_seqlens);
    v.tok_pos = p.at(p.tok_pos);
    v.tok_seq = p.at(p.tok_seq);
    v.tokens = p.at(p.tokens);
    v.want_rows = p.at(p.want_rows);
    v.rows = o.rows == PICOLM_ROWS_STEP ? p.T : p.n_want;
    if (o.in >= 0) {
        v.in = r.buf(o.in);
        v.in_row_bytes = e->buffers[o.in].row_bytes;
    }
    v.out = r.buf(o.out);
    v.out_row_bytes = e->buffers[o.out].row_bytes;
    for (int x = 0; x < 4; ++x)
        if (o.extra[x] >= 0) {
            v.extra[x] = r.buf(o.extra[x]);
            v.extra_row_bytes[x] = e->buffers[o.extra[x]].row_bytes;
        }
    if (o.call_flags & PICOLM_CALL_KV) {
        const KVGroup& g = e->kv[o.kv_group];
        v.k_pages = g.k + (size_t)o.kv_entry * g.k_entry_bytes;
        v.v_pages = g.v + (size_t)o.kv_entry * g.v_entry_bytes;
        v.page_table = g.table_dev;
        v.n_pages = std::max(g.n_pages, 1);
        v.max_pages = g.max_pages;
        v.ring_pages = g.ring_pages;
        v.n_kv_heads = g.spec.n_kv_heads;
        v.head_dim = g.spec.head_dim;
        v.v_head_dim = g.value_dim();
        v.window = g.spec.window;
        v.kv_writes = o.kv_writes;
        if (o.kv_writes) v.write_pages = p.at(p.write_pages[o.kv_group]);
        if (o.call_flags & PICOLM_CALL_ATTENDS) {
            if (p.is_decode) {
                const DecodeList& l = p.lists[o.kv_group];
                v.chunk_list = p.at(l.span);
                v.n_chunks = l.n_chunks;
                v.pages_per_chunk = p.pages_per_chunk;
                v.most_chunks = l.most;
                v.partial = l.most > 1 && o.partial_floats ? (float*)(r.w.base + r.w.partial) : nullptr;
                v.counters = r.w.counters;
            } else if (o.tile_rows > 0) {
                const TileList* tl = p.tiles_of(o.tile_rows);
                E_REQUIRE(-1, tl != nullptr, "call: the step has no tiles of %d rows", o.tile_rows);
                v.tile_seq = p.at(tl->seq);
                v.tile_q0 = p.at(tl->q0);
                v.n_tiles = tl->n;
                v.tile_rows = o.tile_rows;
            }
        }
    }
    if (o.call_flags & PICOLM_CALL_STATE) {
        const StateGroup& sg = e->state[o.state_group];
        v.state = sg.data + (size_t)o.state_entry * e->n_slots * sg.spec.bytes_per_slot;
        v.state_bytes_per_slot = sg.spec.bytes_per_slot;
    }
    v.n_slots = e->n_slots;
    v.stream = r.stream;
    const int rc = o.call(o.call_user, &v);
    if (rc == 0) return 0;
    return rc == PICOLM_ERR_STEP || rc == PICOLM_ERR_CACHE_FULL || rc == PICOLM_ERR_CACHE || rc == PICOLM_ERR_DEVICE || rc == -1 || rc == -2
               ? rc
               : PICOLM_ERR_STEP;
}

// embedding -> the layer calls -> final norm on the wanted rows -> head
// (picolm/model_core.c:1785, :1799-2210, :2213, :2220), as the program lists them.
static int timing_event(picolm_engine* e, hipEvent_t* ev, hipStream_t stream) {
    if (!e->spare_events.empty()) {
        *ev = e->spare_events.back();
        e->spare_events.pop_back();
    } else {
        HIP_TRY(hipEventCreate(ev));
    }
    HIP_TRY(hipEventRecord(*ev, stream));
    return 0;
}

static int run_program(picolm_engine* e, const StepPlan& p, Workspace& w, hipStream_t stream) {
    Run r{e, p, w, stream, Prepared()};
    for (const picolm_op& o : e->ops) {
        if (o.rows == PICOLM_ROWS_WANTED && p.n_want == 0) continue;
        hipEvent_t before = nullptr;
        if (e->timing()) TRY(timing_event(e, &before, stream));
        switch (o.kind) {
            case PICOLM_OP_EMBED:
                TRY(picolm_embed(o.weight, o.weight_dt, p.at(p.tokens), (float*)r.buf(o.out), p.T, o.k, o.n, stream));
                break;
            case PICOLM_OP_RMSNORM: {
                r.prepared = Prepared();
                const bool all_rows = o.rows == PICOLM_ROWS_STEP || p.every_row;
                TRY(picolm_rmsnorm((const float*)r.buf(o.in), (const float*)o.weight, r.buf(o.out), e->buffers[o.out].dtype,
                                   all_rows ? nullptr : p.at(p.want_rows), o.rows == PICOLM_ROWS_STEP ? p.T : p.n_want, o.k, o.eps, stream));
                break;
            }
            case PICOLM_OP_LINEAR: TRY(run_linear(r, o)); break;
            case PICOLM_OP_ATTENTION: TRY(run_attention(r, o)); break;
            case PICOLM_OP_CALL: TRY(run_call(r, o)); break;
        }
        // what a product prepared of a norm holds for the rows as they were: whoever writes them since
        // (any operation but the product that just prepared it) makes it stale
        if (r.prepared.x == r.buf(o.out) && !(o.kind == PICOLM_OP_LINEAR && r.prepared.by == &o)) r.prepared = Prepared();
        if (o.kind == PICOLM_OP_CALL) r.prepared = Prepared();      // (it may write any of its buffers)
        if (e->timing()) {
            hipEvent_t after = nullptr;
            TRY(timing_event(e, &after, stream));
            const int cls = o.kind == PICOLM_OP_LINEAR ? (o.rows == PICOLM_ROWS_WANTED ? 2 : 1) : o.kind == PICOLM_OP_ATTENTION ? 3 : 0;
            e->timed.push_back({cls, before, after});
        }
    }
    return 0;
}

extern "C" int picolm_engine_op_times(picolm_engine* e, double* ms) {
    E_REQUIRE(-1, e && ms && e->timing(), "op_times: the engine was not made with PICOLM_ENGINE_TIME_OPS");
    for (int c = 0; c < 4; ++c) ms[c] = 0.0;
    for (auto& t : e->timed) {
        HIP_TRY(hipEventSynchronize(t.after));
        float dt = 0.f;
        HIP_TRY(hipEventElapsedTime(&dt, t.before, t.after));
        ms[t.cls] += dt;
        e->spare_events.push_back(t.before);
        e->spare_events.push_back(t.after);
    }
    e->timed.clear();
    return 0;
}

// ---- the step ------------------------------------------------------------------------------------
static int check_sequences(picolm_engine* e, int n_seq, const int32_t* slots, std::vector<int>& sl, std::vector<int>& pos0) {
    E_REQUIRE(PICOLM_ERR_STEP, n_seq > 0, "a step needs at least one sequence");
    E_REQUIRE(-1, slots != nullptr, "step: null slots");
    sl.assign(slots, slots + n_seq);
    std::vector<char> seen(e->n_slots, 0);
    pos0.resize(n_seq);
    for (int i = 0; i < n_seq; ++i) {
        E_REQUIRE(PICOLM_ERR_STEP, e->slots.is_live(sl[i]), "slot %d is not live", sl[i]);
        E_REQUIRE(PICOLM_ERR_STEP, !seen[sl[i]], "a slot appears twice in one step (slot %d)", sl[i]);
        seen[sl[i]] = 1;
        pos0[i] = e->slots.length[sl[i]];
    }
    return 0;
}

static int decode_step(picolm_engine* e, const std::vector<int>& slots, const std::vector<int>& pos0, const int32_t* tokens,
                       const int32_t* tokens_dev, float** logits, hipStream_t stream) {
    const int n = (int)slots.size();
    std::vector<int> lengths(n);
    for (int i = 0; i < n; ++i) lengths[i] = pos0[i] + 1;
    TRY(reserve_many(e, slots, lengths));
    TRY(flush_tables(e, stream));
    const int ppc = decode_pages_per_chunk(pos0, e->decode_blocks_per_chunk, e->decode_max_pages_per_chunk);
    // the step's shape: the chunks that the longest sequence needs, rounded up to a power of two, so
    // that a launch covers what the live contexts need and not what the cache could hold
    int need = 1, most_chunks = 1;
    for (size_t gi = 0; gi < e->kv.size(); ++gi)
        if (e->group_attended[gi])
            for (int q : pos0) need = std::max(need, chunks_of(e->kv[gi], q, ppc));
    while (most_chunks < need) most_chunks *= 2;
    const auto key = std::make_tuple(n, ppc, most_chunks);
    auto& slot = e->graphs[key];
    if (!slot) {
        slot.reset(new DecodeGraph);
        const int rc = decode_batch_init(e, slot->batch, n, ppc, most_chunks);
        if (rc) {
            e->graphs.erase(key);
            return rc;
        }
        if (e->graphs.size() > MAX_DECODE_SHAPES) {
            auto oldest = e->graphs.end();
            for (auto it = e->graphs.begin(); it != e->graphs.end(); ++it)
                if (it->first != key && (oldest == e->graphs.end() || it->second->last_used < oldest->second->last_used)) oldest = it;
            if (!e->host_only()) HIP_TRY(hipStreamSynchronize(stream));      // its last step may still read its block
            free_decode_graph(e, *oldest->second);
            e->graphs.erase(oldest);
        }
    }
    DecodeGraph& g = *e->graphs[key];
    g.last_used = ++e->decode_tick;
    TRY(decode_batch_fill(e, g.batch, slots, pos0, tokens, stream));
    e->last_plan = &g.batch.plan;
    if (!e->host_only()) {
        const StepPlan& p = g.batch.plan;
        Workspace& ws = e->decode_ws;
        if (tokens_dev)
            HIP_TRY(hipMemcpyAsync(g.batch.dev + p.tokens.off, tokens_dev, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
        g.uses++;
        int most = 1;
        for (auto& l : p.lists) most = std::max(most, l.most);
        TRY(workspace_ensure(e, ws, p, most));
        if (g.exec && g.ws_generation != ws.generation) {      // the workspace has moved since the recording
            (void)hipGraphExecDestroy(g.exec);
            g.exec = nullptr;
        }
        if (g.exec) {
            HIP_TRY(hipGraphLaunch(g.exec, stream));
        } else {
            TRY(run_program(e, p, ws, stream));
            if (g.uses >= 2 && e->recordable && !(e->flags & (PICOLM_ENGINE_NO_GRAPHS | PICOLM_ENGINE_TIME_OPS))) {
                // the sizes have been seen and the workspace is allocated: record the same launches
                // (recording runs nothing; this step's result came from the launches above)
                hipGraph_t graph = nullptr;
                const int flip = ws.flip;
                HIP_TRY(hipStreamBeginCapture(e->capture_stream, hipStreamCaptureModeThreadLocal));
                const int rc = run_program(e, p, ws, e->capture_stream);
                const hipError_t end = hipStreamEndCapture(e->capture_stream, &graph);
                ws.flip = flip;
                if (rc) {
                    if (graph) (void)hipGraphDestroy(graph);
                    return rc;
                }
                HIP_TRY(end);
                const hipError_t inst = hipGraphInstantiate(&g.exec, graph, nullptr, nullptr, 0);
                (void)hipGraphDestroy(graph);
                HIP_TRY(inst);
                g.ws_generation = ws.generation;
            }
        }
        if (logits) *logits = (float*)(ws.base + ws.offsets[e->logits_buffer]);
    }
    for (int i = 0; i < n; ++i) e->slots.length[slots[i]] = pos0[i] + 1;
    return 0;
}

extern "C" int picolm_engine_step(picolm_engine* e, int32_t n_seq, const int32_t* slots, const int32_t* n_new, const int32_t* tokens,
                                  const int32_t* want_counts, const int32_t* want, float** logits, int32_t* n_rows,
                                  hipStream_t stream) {
    E_REQUIRE(-1, e != nullptr, "step: null engine");
    std::vector<int> sl, pos0;
    TRY(check_sequences(e, n_seq, slots, sl, pos0));
    E_REQUIRE(-1, n_new && tokens, "step: null token counts or tokens");
    std::vector<int> nn(n_new, n_new + n_seq), lengths(n_seq);
    int64_t T = 0;
    for (int i = 0; i < n_seq; ++i) {
        E_REQUIRE(PICOLM_ERR_STEP, nn[i] >= 1, "every sequence of a step brings at least one token");
        T += nn[i];
        lengths[i] = pos0[i] + nn[i];
    }
    E_REQUIRE(PICOLM_ERR_STEP, T < (1ll << 30), "a step of %lld tokens", (long long)T);
    for (int64_t t = 0; t < T; ++t)
        E_REQUIRE(PICOLM_ERR_STEP, tokens[t] >= 0 && tokens[t] < e->vocab, "token id %d is outside the vocabulary of %d", tokens[t], e->vocab);
    std::vector<std::vector<int>> wanted(n_seq);
    bool last_of_each = true;
    if (want_counts) {
        E_REQUIRE(-1, want != nullptr, "step: wanted rows are counted but not listed");
        int64_t off = 0;
        for (int i = 0; i < n_seq; ++i) {
            E_REQUIRE(PICOLM_ERR_STEP, want_counts[i] >= 0, "sequence %d wants %d rows", i, want_counts[i]);
            for (int j = 0; j < want_counts[i]; ++j) {
                const int w = want[off + j];
                E_REQUIRE(PICOLM_ERR_STEP, w >= 0 && w < nn[i], "wanted row %d of a sequence that brings %d tokens", w, nn[i]);
                wanted[i].push_back(w);
            }
            off += want_counts[i];
            last_of_each = last_of_each && want_counts[i] == 1 && wanted[i][0] == nn[i] - 1;
        }
    } else {
        for (int i = 0; i < n_seq; ++i) wanted[i].push_back(nn[i] - 1);
    }
    if (n_rows) {
        *n_rows = 0;
        for (auto& w : wanted) *n_rows += (int)w.size();
    }
    if (T == n_seq && last_of_each) return decode_step(e, sl, pos0, tokens, nullptr, logits, stream);
    // A ring holds a window and WINDOW_STEP_TOKENS new tokens.  The ATTENTION operation writes and
    // answers a longer prompt slice by slice; a called operation sees the step as a whole.
    if (e->call_on_ring)
        for (int i = 0; i < n_seq; ++i)
            E_REQUIRE(PICOLM_ERR_STEP, nn[i] <= WINDOW_STEP_TOKENS,
                      "a called operation on a cache group with a window takes steps of up to %d tokens a sequence, sequence %d brings %d",
                      WINDOW_STEP_TOKENS, i, nn[i]);
    TRY(reserve_many(e, sl, lengths));
    TRY(flush_tables(e, stream));
    plan_step(e, e->plan, sl, pos0, nn, tokens, wanted);
    e->last_plan = &e->plan;
    if (!e->host_only()) {
        TRY(upload_plan(e, e->plan, stream));
        int most = 1;
        for (auto& l : e->plan.lists) most = std::max(most, l.most);
        TRY(workspace_ensure(e, e->ws, e->plan, most));
        TRY(run_program(e, e->plan, e->ws, stream));
        if (logits) *logits = (float*)(e->ws.base + e->ws.offsets[e->logits_buffer]);
    }
    for (int i = 0; i < n_seq; ++i) e->slots.length[sl[i]] = lengths[i];
    return 0;
}

extern "C" int picolm_engine_step_device_tokens(picolm_engine* e, int32_t n_seq, const int32_t* slots, const int32_t* tokens_dev,
                                                float** logits, hipStream_t stream) {
    E_REQUIRE(-1, e != nullptr && tokens_dev != nullptr, "step: null engine or tokens");
    E_REQUIRE(-1, !e->host_only(), "step: an engine without device memory takes its tokens from the host");
    std::vector<int> sl, pos0;
    TRY(check_sequences(e, n_seq, slots, sl, pos0));
    return decode_step(e, sl, pos0, nullptr, tokens_dev, logits, stream);
}

// ---- what the engine holds -----------------------------------------------------------------------
extern "C" int64_t picolm_engine_info(picolm_engine* e, int32_t what) {
    if (!e) return -1;
    switch (what) {
        case 0: return e->max_seq_len;
        case 1: return e->n_slots;
        case 2: return (int64_t)e->slots.free_.size();
        case 3: {
            if (e->kv.empty()) return (int64_t)1 << 40;       // a model without keys and values has no pages to run out of
            int64_t free_pages = -1;
            for (const KVGroup& g : e->kv) free_pages = free_pages < 0 ? g.pool.n_free() : std::min<int64_t>(free_pages, g.pool.n_free());
            return std::max<int64_t>(free_pages, 0) * PAGE_TOKENS;
        }
        case 4: {
            int64_t n = 0;
            for (auto& g : e->graphs) n += g.second->exec != nullptr;
            return n;
        }
        case 5: return e->max_pages;
        case 6: return (int64_t)e->device_bytes;
        case 7: return e->version;
        case 8: return e->call_on_ring ? WINDOW_STEP_TOKENS : 0;
        case 9: {
            int64_t bytes = 0;
            for (const KVGroup& g : e->kv) bytes += (int64_t)(g.k_entry_bytes + g.v_entry_bytes) * g.spec.n_entries;
            for (const StateGroup& s : e->state) bytes += (int64_t)s.spec.n_entries * e->n_slots * s.spec.bytes_per_slot;
            return bytes;
        }
    }
    return -1;
}

extern "C" int picolm_engine_kv_entry(picolm_engine* e, int32_t group, int32_t entry, void** k, void** v, int64_t* n_pages) {
    E_REQUIRE(-1, e && group >= 0 && group < (int)e->kv.size(), "kv_entry: no cache group %d", group);
    const KVGroup& g = e->kv[group];
    E_REQUIRE(-1, entry >= 0 && entry < g.spec.n_entries, "kv_entry: group %d has %d entries", group, g.spec.n_entries);
    if (k) *k = g.k ? g.k + (size_t)entry * g.k_entry_bytes : nullptr;
    if (v) *v = g.v ? g.v + (size_t)entry * g.v_entry_bytes : nullptr;
    if (n_pages) *n_pages = std::max(g.n_pages, 1);
    return 0;
}

extern "C" int picolm_engine_state_entry(picolm_engine* e, int32_t group, int32_t entry, void** state, int64_t* bytes_per_slot) {
    E_REQUIRE(-1, e && group >= 0 && group < (int)e->state.size(), "state_entry: no state group %d", group);
    const StateGroup& s = e->state[group];
    E_REQUIRE(-1, entry >= 0 && entry < s.spec.n_entries, "state_entry: group %d has %d entries", group, s.spec.n_entries);
    if (state) *state = s.data ? s.data + (size_t)entry * e->n_slots * s.spec.bytes_per_slot : nullptr;
    if (bytes_per_slot) *bytes_per_slot = s.spec.bytes_per_slot;
    return 0;
}

extern "C" int picolm_engine_slot_pages(picolm_engine* e, int32_t group, int32_t slot, int32_t* pages, int32_t capacity) {
    E_REQUIRE(-1, e && group >= 0 && group < (int)e->kv.size() && slot >= 0 && slot < e->n_slots, "slot_pages: no group %d or slot %d", group, slot);
    const auto& held = e->kv[group].pages[slot];
    for (int i = 0; i < (int)held.size() && i < capacity && pages; ++i) pages[i] = held[i];
    return (int)held.size();
}

extern "C" int picolm_engine_free_pages(picolm_engine* e, int32_t group) {
    E_REQUIRE(-1, e && group >= 0 && group < (int)e->kv.size(), "free_pages: no cache group %d", group);
    return e->kv[group].pool.n_free();
}

extern "C" int picolm_engine_step_array(picolm_engine* e, const char* name, int32_t* out, int32_t capacity) {
    E_REQUIRE(-1, e && name && e->last_plan, "step_array: no step has been planned");
    const StepPlan& p = *e->last_plan;
    const std::string n(name);
    Span s;
    bool found = true;
    if (n == "seq_slot") s = p.seq_slot;
    else if (n == "seq_pos0") s = p.seq_pos0;
    else if (n == "seq_nnew") s = p.seq_nnew;
    else if (n == "cu_seqlens") s = p.cu_seqlens;
    else if (n == "tok_pos") s = p.tok_pos;
    else if (n == "tok_seq") s = p.tok_seq;
    else if (n == "tokens") s = p.tokens;
    else if (n == "want_rows") s = p.want_rows;
    else if (n.rfind("write_pages.", 0) == 0) {
        const int g = atoi(n.c_str() + 12);
        found = g >= 0 && g < (int)p.write_pages.size() && p.write_pages[g].n > 0;
        if (found) s = p.write_pages[g];
    } else if (n.rfind("chunks.", 0) == 0) {
        const int g = atoi(n.c_str() + 7);
        found = g >= 0 && g < (int)p.lists.size() && p.lists[g].span.n > 0;
        if (found) s = p.lists[g].span;
    } else if (n.rfind("window_chunk.", 0) == 0) {
        // "window_chunk.<c>.<array>": a slice of a prefill step for the groups that keep a ring
        const int c = atoi(n.c_str() + 13);
        const size_t dot = n.find('.', 13);
        found = c >= 0 && c < (int)p.window_chunks.size() && dot != std::string::npos;
        if (found) {
            const WindowChunk& wc = p.window_chunks[c];
            const std::string what = n.substr(dot + 1);
            if (what == "seq_slot") s = wc.seq_slot;
            else if (what == "seq_pos0") s = wc.seq_pos0;
            else if (what == "seq_nnew") s = wc.seq_nnew;
            else if (what == "first_row") s = wc.first_row;
            else if (what == "rows") s = wc.rows;
            else if (what.rfind("tiles.", 0) == 0) {
                const TileList* tl = wc.tiles_of(atoi(what.c_str() + 6));
                found = tl != nullptr;
                if (found) s = what.find(".seq") != std::string::npos ? tl->seq : tl->q0;
            } else {
                found = false;
            }
        }
    } else if (n.rfind("tiles.", 0) == 0) {
        const int rows = atoi(n.c_str() + 6);
        const TileList* tl = p.tiles_of(rows);
        found = tl != nullptr;
        if (found) s = n.find(".seq") != std::string::npos ? tl->seq : tl->q0;
    } else {
        found = false;
    }
    E_REQUIRE(-1, found, "step_array: the step planned last has no array '%s'", name);
    for (int i = 0; i < s.n && i < capacity && out; ++i) out[i] = p.ints[s.off + i];
    return s.n;
}

extern "C" int picolm_engine_set_prefill_step_tokens(picolm_engine* e, int32_t tokens) {
    E_REQUIRE(-1, e && tokens >= 64, "prefill_step_tokens: at least one page of 64 tokens");
    e->prefill_step_tokens = tokens;
    return 0;
}

// ---- generation ------------------------------------------------------------------------------------
// Initial xorshift64 state of sequence `index`: sequence 0 has picolm's single stream
// (`seed ? seed : 42`, picolm/sampler.c:43); the others are offset so that a sequence's draws do
// not depend on what else is in its batch.
static uint64_t stream_state(uint64_t seed, uint64_t index) {
    uint64_t s = seed ? seed : 42;
    s += index * 0x9E3779B97F4A7C15ull;
    return s ? s : 42;
}

static int gen_buffers(picolm_engine* e, int n_prompts, int rows, const picolm_sampling* sp) {
    if (rows > e->gen_rows) {
        if (e->gen_tokens_dev) HIP_TRY(hipFree(e->gen_tokens_dev));
        if (e->gen_tokens_host) HIP_TRY(hipHostFree(e->gen_tokens_host));
        if (e->gen_index) HIP_TRY(hipFree(e->gen_index));
        HIP_TRY(hipMalloc((void**)&e->gen_tokens_dev, (size_t)rows * 4 * 4));
        HIP_TRY(hipHostMalloc((void**)&e->gen_tokens_host, (size_t)rows * 4 * 2, hipHostMallocDefault));
        HIP_TRY(hipMalloc((void**)&e->gen_index, (size_t)rows * 4));
        e->gen_rows = rows;
    }
    for (int t = 0; t < 2; ++t)
        if (!e->gen_arrived[t]) HIP_TRY(hipEventCreateWithFlags(&e->gen_arrived[t], hipEventDisableTiming));
    if (e->gen_states) HIP_TRY(hipFree(e->gen_states));
    e->gen_states = nullptr;
    std::vector<uint64_t> states(n_prompts);
    for (int i = 0; i < n_prompts; ++i) states[i] = stream_state(sp->seed, (uint64_t)i);
    HIP_TRY(hipMalloc((void**)&e->gen_states, (size_t)n_prompts * 8));
    HIP_TRY(hipMemcpy(e->gen_states, states.data(), (size_t)n_prompts * 8, hipMemcpyHostToDevice));
    const size_t need = sp->temperature > 0.f ? (size_t)picolm_sample_scratch_bytes(rows, e->vocab, sp->temperature, sp->top_k)
                                              : (size_t)picolm_argmax_scratch_floats(rows, e->vocab) * 4;
    if (need > e->gen_scratch_bytes) {
        if (e->gen_scratch) HIP_TRY(hipFree(e->gen_scratch));
        HIP_TRY(hipMalloc(&e->gen_scratch, need));
        e->gen_scratch_bytes = need;
    }
    return 0;
}

// One token for each row of logits; row i belongs to request ids[i].  The draw and the tokens' way
// to the host are queued, nothing is waited for: the tokens lie in gen_tokens_dev + turn * gen_rows
// when the stream gets there and in gen_tokens_host + turn * gen_rows after gen_wait(turn).
static int gen_draw(picolm_engine* e, const float* logits, const std::vector<int>& ids, const picolm_sampling* sp, int turn,
                    hipStream_t stream) {
    const int n = (int)ids.size();
    int32_t* out = e->gen_tokens_dev + (size_t)turn * e->gen_rows;
    if (sp->temperature > 0.f) {
        TRY(e->stager.upload(e->gen_index, ids.data(), (size_t)n * 4, stream));
        const int64_t scratch = picolm_sample_scratch_bytes(n, e->vocab, sp->temperature, sp->top_k);
        TRY(picolm_sample(logits, e->vocab, n, e->vocab, sp->temperature, sp->top_k, sp->top_p, sp->min_p, e->gen_states, e->gen_index,
                          out, scratch ? e->gen_scratch : nullptr, scratch, stream));
    } else {
        TRY(picolm_argmax(logits, out, n, e->vocab, e->vocab, (float*)e->gen_scratch, stream));
    }
    HIP_TRY(hipMemcpyAsync(e->gen_tokens_host + (size_t)turn * e->gen_rows, out, (size_t)n * 4, hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipEventRecord(e->gen_arrived[turn], stream));
    return 0;
}
static int gen_wait(picolm_engine* e, int turn, const int32_t** tokens) {
    HIP_TRY(hipEventSynchronize(e->gen_arrived[turn]));
    *tokens = e->gen_tokens_host + (size_t)turn * e->gen_rows;
    return 0;
}

extern "C" int picolm_engine_generate(picolm_engine* e, int32_t n_prompts, const int32_t* prompts, const int32_t* prompt_lens,
                                      int32_t max_new, const picolm_sampling* sampling, const int32_t* stop_ids, int32_t n_stop,
                                      int32_t batch_size, int32_t* out_tokens, int32_t* out_counts, int32_t* out_finish,
                                      hipStream_t stream) {
    E_REQUIRE(-1, e && !e->host_only(), "generate: needs an engine with device memory");
    E_REQUIRE(-1, n_prompts >= 0 && (n_prompts == 0 || (prompts && prompt_lens && out_tokens && out_counts && out_finish)) && sampling,
              "generate: null argument");
    E_REQUIRE(-1, sampling->top_k >= 0 && sampling->top_p > 0.f && sampling->min_p >= 0.f, "generate: top_k %d, top_p %g, min_p %g",
              sampling->top_k, sampling->top_p, sampling->min_p);
    batch_size = std::max(1, batch_size);
    std::vector<int64_t> start(n_prompts + 1, 0);
    for (int i = 0; i < n_prompts; ++i) {
        E_REQUIRE(PICOLM_ERR_STEP, prompt_lens[i] >= 1, "request %d has an empty prompt; give at least a start token", i);
        E_REQUIRE(PICOLM_ERR_STEP, prompt_lens[i] <= e->max_seq_len, "request %d has %d prompt tokens, the cache takes %d", i,
                  prompt_lens[i], e->max_seq_len);
        start[i + 1] = start[i] + prompt_lens[i];
        out_counts[i] = 0;
        out_finish[i] = 0;
    }
    if (n_prompts == 0) return 0;
    TRY(gen_buffers(e, n_prompts, std::min(batch_size, n_prompts), sampling));
    auto is_stop = [&](int tok) {
        for (int j = 0; j < n_stop; ++j)
            if (stop_ids[j] == tok) return true;
        return false;
    };
    int first = 0;
    while (first < n_prompts) {
        // admission: as many requests as the free slots and pages hold at their full lengths
        int n = 0;
        int64_t pages = 0;
        const int64_t free_pages = picolm_engine_info(e, 3) / PAGE_TOKENS;
        while (first + n < n_prompts && n < batch_size && n < (int)e->slots.free_.size()) {
            const int need = pages_for(std::min<int64_t>((int64_t)prompt_lens[first + n] + max_new, e->max_seq_len));
            if (!e->kv.empty() && pages + need > free_pages) break;
            pages += need;
            ++n;
        }
        E_REQUIRE(PICOLM_ERR_CACHE_FULL, n > 0, "request %d (%d prompt tokens, %d new) does not fit the cache even alone", first,
                  prompt_lens[first], max_new);
        std::vector<int> ids(n), slot_of(n_prompts, -1), length(n_prompts, 0);
        int rc = 0;
        for (int i = 0; i < n && !rc; ++i) {
            ids[i] = first + i;
            int32_t s = -1;
            rc = picolm_engine_slot_alloc(e, &s, stream);
            slot_of[first + i] = s;
            length[first + i] = prompt_lens[first + i];
        }
        auto release_all = [&]() {
            for (int i = first; i < first + n; ++i)
                if (slot_of[i] >= 0) {
                    (void)picolm_engine_slot_free(e, slot_of[i]);
                    slot_of[i] = -1;
                }
        };
        if (rc) {
            release_all();
            return rc;
        }
        if (max_new <= 0) {
            for (int i : ids) out_finish[i] = 2;
            release_all();
            first += n;
            continue;
        }
        // what a sampled token means for its request: recorded; the request goes on or ends and
        // gives its slot back at once
        std::vector<int> last_token(n_prompts, 0);
        auto accept = [&](int i, int tok) {
            out_tokens[(int64_t)i * max_new + out_counts[i]++] = tok;
            last_token[i] = tok;
            if (is_stop(tok)) out_finish[i] = 1;
            else if (out_counts[i] >= max_new) out_finish[i] = 2;
            else if (length[i] + 1 > e->max_seq_len) out_finish[i] = 3;
            else return true;
            (void)picolm_engine_slot_free(e, slot_of[i]);
            slot_of[i] = -1;
            return false;
        };
        // the prompts: one step if they fit the step's token budget, else several, each giving every
        // unfinished prompt an equal share in whole pages; a prompt's last step gives its first token
        std::vector<int> done(n, 0), live;
        std::vector<int32_t> sl, nn, toks, counts, idx;
        float* logits = nullptr;
        int64_t total = 0;
        for (int i = 0; i < n; ++i) total += prompt_lens[ids[i]];
        while (!rc) {
            std::vector<int> left;
            for (int i = 0; i < n; ++i)
                if (done[i] < prompt_lens[ids[i]]) left.push_back(i);
            if (left.empty()) break;
            const int budget = e->prefill_step_tokens;
            int share = total <= budget ? (1 << 30) : std::max(64, budget / (int)left.size() / 64 * 64);
            if (e->call_on_ring) share = std::min(share, WINDOW_STEP_TOKENS);      // what such a step may bring a sequence
            int64_t room = total <= budget ? total : std::max<int64_t>(budget, 64 * (int64_t)left.size());
            sl.clear(), nn.clear(), toks.clear(), counts.clear(), idx.clear();
            std::vector<int> ending;
            for (int i : left) {
                const int id = ids[i];
                const int take = (int)std::min<int64_t>(std::min(prompt_lens[id] - done[i], share), room);
                if (take <= 0) continue;
                sl.push_back(slot_of[id]);
                nn.push_back(take);
                toks.insert(toks.end(), prompts + start[id] + done[i], prompts + start[id] + done[i] + take);
                done[i] += take;
                room -= take;
                const bool ends = done[i] == prompt_lens[id];
                counts.push_back(ends ? 1 : 0);
                if (ends) {
                    idx.push_back(take - 1);
                    ending.push_back(id);
                }
            }
            if (idx.empty()) idx.push_back(0);
            rc = picolm_engine_step(e, (int)sl.size(), sl.data(), nn.data(), toks.data(), counts.data(), idx.data(), &logits, nullptr, stream);
            if (rc || ending.empty()) continue;
            const int32_t* drawn = nullptr;
            rc = gen_draw(e, logits, ending, sampling, 0, stream);
            if (!rc) rc = gen_wait(e, 0, &drawn);
            for (size_t x = 0; !rc && x < ending.size(); ++x)
                if (accept(ending[x], drawn[x])) live.push_back(ending[x]);
        }
        std::sort(live.begin(), live.end());
        // Decoding, one step ahead of the host: the step that takes the tokens of a draw is queued
        // before those tokens have been read here.  Whether a sequence ends by its count of tokens
        // or at the cache's capacity is known without its token; only a stop token is found out one
        // step late, and such a sequence has by then been stepped once more (that step's token is
        // dropped; its slot is given back at once: what still runs for it touches its own pages
        // only, and whatever uses them next comes after it in the stream).
        std::vector<int> rows;               // the sequences that the pending tokens belong to, row by row
        int turn = 0;
        if (!rc && !live.empty()) {          // the first step takes its tokens from the host
            sl.resize(live.size());
            nn.assign(live.size(), 1);
            toks.resize(live.size());
            for (size_t x = 0; x < live.size(); ++x) {
                sl[x] = slot_of[live[x]];
                toks[x] = last_token[live[x]];
                length[live[x]] += 1;
            }
            rc = picolm_engine_step(e, (int)live.size(), sl.data(), nn.data(), toks.data(), nullptr, nullptr, &logits, nullptr, stream);
            if (!rc) rc = gen_draw(e, logits, live, sampling, turn, stream);
            if (!rc) rows = live;
        }
        std::vector<char> ended(n_prompts, 0);
        while (!rc && !rows.empty()) {
            std::vector<int> ahead, pick;
            for (size_t x = 0; x < rows.size(); ++x) {
                const int i = rows[x];
                if (!ended[i] && out_counts[i] + 1 < max_new && length[i] + 1 <= e->max_seq_len) {
                    ahead.push_back(i);
                    pick.push_back((int)x);
                }
            }
            if (!ahead.empty()) {
                const int32_t* step_tokens = e->gen_tokens_dev + (size_t)turn * e->gen_rows;
                if (ahead.size() != rows.size()) {       // a smaller batch goes on: its tokens, picked on the device
                    int32_t* picked = e->gen_tokens_dev + (size_t)2 * e->gen_rows;
                    int32_t* index = e->gen_tokens_dev + (size_t)3 * e->gen_rows;
                    rc = e->stager.upload(index, pick.data(), pick.size() * 4, stream);
                    if (!rc) rc = picolm_gather_i32(picked, step_tokens, index, (int)pick.size(), stream);
                    step_tokens = picked;
                }
                sl.resize(ahead.size());
                for (size_t x = 0; x < ahead.size(); ++x) sl[x] = slot_of[ahead[x]];
                if (!rc) rc = picolm_engine_step_device_tokens(e, (int)ahead.size(), sl.data(), step_tokens, &logits, stream);
                if (!rc) rc = gen_draw(e, logits, ahead, sampling, turn ^ 1, stream);
                if (rc) break;
                for (int i : ahead) length[i] += 1;
            }
            const int32_t* drawn = nullptr;
            rc = gen_wait(e, turn, &drawn);
            if (rc) break;
            for (size_t x = 0; x < rows.size(); ++x) {
                const int i = rows[x];
                if (ended[i]) continue;                  // stepped once more before its stop token was seen
                const int tok = drawn[x];
                out_tokens[(int64_t)i * max_new + out_counts[i]++] = tok;
                if (is_stop(tok)) out_finish[i] = 1;
                else if (std::find(ahead.begin(), ahead.end(), i) != ahead.end()) continue;
                else out_finish[i] = out_counts[i] >= max_new ? 2 : 3;
                ended[i] = 1;
                (void)picolm_engine_slot_free(e, slot_of[i]);
                slot_of[i] = -1;
            }
            rows = ahead;
            turn ^= 1;
        }
        release_all();
        if (rc) return rc;
        first += n;
    }
    return 0;
}
