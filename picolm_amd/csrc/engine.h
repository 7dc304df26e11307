// The engine behind a C ABI: a cache with a slot per sequence, the step function and a generation
// loop, for a model given as a launch program.
//
// picolm's counterpart is model_load / model_forward / model_forward_prefill / model_free
// (picolm/model.h:504-551) and sampler_init / sampler_sample (picolm/sampler.h:14-16): one
// sequence, one architecture's layer order written out in C.  Here the layer order is data.  A
// model is a flat list of operations over named row buffers (a "program"), which the parts of a
// model emit once (picolm_amd/parts/*.py, `emit`); the engine owns everything that changes from
// step to step: slots and pages, the step's index arrays, the workspace, recorded decode steps.
// Weights stay with the caller, as device pointers inside the operations.
//
// A program is made by whoever knows the architecture: in this library the Python parts read
// config.json, bind the checkpoint's tensors and emit it (picolm_amd/engine/model.py), so a C
// caller starts at a built program, where picolm's starts at a file name (model_load).  The set
// of operations is open: PICOLM_OP_CALL hands the running step to a function of the caller's, so
// that a part with kernels of its own (a mixer with state, another norm, a routed feed-forward)
// joins a program without a change to this header or to the engine.
//
// Every function returns 0 or a negative code and leaves a message for picolm_last_error().
// Nothing here waits for the GPU unless it says so; work is queued on the stream that is passed
// in, and all calls on one engine must use one stream (or be ordered by the caller).  An engine is
// used by one thread at a time.
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

// return codes beside -1 (bad argument) and -2 (a launch failed)
#define PICOLM_ERR_STEP (-10)        // a step that cannot run: a dead slot, a token outside the vocabulary
#define PICOLM_ERR_CACHE_FULL (-11)  // no free slot or page, or a sequence longer than the cache takes
#define PICOLM_ERR_CACHE (-12)       // a slot freed twice, a slot that does not exist
#define PICOLM_ERR_DEVICE (-13)      // the HIP runtime refused something

enum { PICOLM_OP_EMBED = 1, PICOLM_OP_RMSNORM = 2, PICOLM_OP_LINEAR = 3, PICOLM_OP_ATTENTION = 4, PICOLM_OP_CALL = 5 };
// which rows of the step an operation covers: every new token's, or only those whose logits are wanted
enum { PICOLM_ROWS_STEP = 0, PICOLM_ROWS_WANTED = 1 };

// A row buffer of the workspace: `row_bytes` bytes for each of the step's rows of that kind.
typedef struct {
    int32_t row_bytes;
    int32_t rows;            // PICOLM_ROWS_STEP or PICOLM_ROWS_WANTED
    int32_t dtype;           // PICOLM_F32 (0) or PICOLM_BF16 (1)
} picolm_buffer;

// What a called operation (PICOLM_OP_CALL) sees of the running step.  Everything is read-only for
// it but the memory behind `out`, `extra` of buffers it writes, its cache entry and its state.
// Host arrays are valid during the call; device memory until the step's work has run.
typedef struct {
    int32_t struct_bytes;        // sizeof(picolm_step_view) in the library that made it
    int32_t dtype;               // the engine's: PICOLM_F32 or PICOLM_BF16
    int32_t n_seq, n_tokens, n_wanted;
    int32_t is_decode;           // every sequence brings one token
    int32_t every_row_wanted;    // the wanted rows are the step's rows, in order
    int32_t recording;           // the stream records (a decode step that will be replayed): the host arrays
                                 // below hold this step's values and will not be seen again
    const int32_t *slots, *pos0, *n_new;     // host, [n_seq]: cache slot, tokens held before the step, new tokens
    // device int32 arrays: per sequence [n_seq] (cu_seqlens [n_seq + 1]), per token [n_tokens], wanted rows [n_wanted]
    const int32_t *seq_slot, *seq_pos0, *seq_nnew, *cu_seqlens, *tok_pos, *tok_seq, *tokens, *want_rows;
    int32_t rows;                // rows the operation covers: n_tokens or n_wanted
    void *in, *out, *extra[4];   // the operation's buffers (null where it names none)
    int32_t in_row_bytes, out_row_bytes, extra_row_bytes[4];
    // the cache entry of the operation (PICOLM_CALL_KV): keys [n_pages][G][64][d], values [n_pages][G][dv][64]
    void *k_pages, *v_pages;
    const int32_t* page_table;   // device [n_slots][max_pages]; logical page j of a slot lies at column j % ring_pages
    int32_t n_pages, max_pages, ring_pages, n_kv_heads, head_dim, v_head_dim, window, kv_writes;
    const int32_t* write_pages;  // device [n_tokens]: the physical page that takes each new token's key and value
    // with PICOLM_CALL_ATTENDS: the decode step's work list over that group's pages (see
    // picolm_attn_decode_generic in api.h), or the prefill step's tiles of `tile_rows` new tokens
    const int32_t* chunk_list;
    int32_t n_chunks, pages_per_chunk, most_chunks;
    float* partial;              // [n_seq][most_chunks][partial_floats] floats for partial results
    int32_t* counters;           // zero when the call starts; whoever uses them leaves them at zero
    const int32_t *tile_seq, *tile_q0;
    int32_t n_tiles, tile_rows;
    // the state entry of the operation (PICOLM_CALL_STATE): [n_slots][state_bytes_per_slot], zeroed when a slot is given out
    void* state;
    int64_t state_bytes_per_slot;
    int32_t n_slots;
    hipStream_t stream;          // queue the work here; do not wait for it
} picolm_step_view;

// Returns 0, or a negative code after picolm_set_error (or any message of its own: a non-zero
// return fails the step with PICOLM_ERR_STEP unless it is one of the codes above).
typedef int (*picolm_call_fn)(void* user, const picolm_step_view* view);

#define PICOLM_CALL_RECORDABLE 1   // what it queues depends on device memory only (not on the view's host arrays,
                                   // not on allocations of its own): a decode step that holds it may be recorded and replayed
#define PICOLM_CALL_KV 2           // it uses the cache entry (kv_group, kv_entry); kv_writes as for ATTENTION
#define PICOLM_CALL_ATTENDS 4      // with PICOLM_CALL_KV: it wants the decode work list and, with tile_rows > 0, the prefill tiles
#define PICOLM_CALL_STATE 8        // it uses the state entry (state_group, state_entry)

// One operation.  Buffers are indices into the program's buffers.  Fields an operation does not
// use are zero.
//   EMBED      out[t] = weight[tokens[t]] widened to float          weight [n][k] of weight_dt
//   RMSNORM    out = in / sqrt(mean(in^2) + eps) * weight           weight float [k]; in float
//   LINEAR     out (=, +=, = silu-gated) in weight^T                weight [n][k]; epilogue 0, 1, 2
//              in_norm_weight: `in` is scratch and the input is rmsnorm(in_norm_x) with that weight
//              and in_norm_eps; the engine either runs the norm into `in` or, where the kernels
//              can, lets the product before and this one compute it between them.
//              out_norm_weight (epilogue 1): the rmsnorm that meets `out` next, so that this
//              product can prepare it; out_norm_when = 1: only in steps that want every row.
//   ATTENTION  in: float rows [(H + 2G) d] of q, k, v; rotates q and k (cos_table, sin_table
//              [table_positions][d/2], null for none; rope_style 0 pairs (2i, 2i+1), 1 pairs
//              (i, i + d/2)), writes k and v to cache entry (kv_group, kv_entry) unless
//              kv_writes = 0, attends over the cache; out [H d]; q_buffer: scratch [H d].
//              window > 0: only the last `window` keys are seen, and the group keeps a ring of pages.
//   CALL       call(call_user, view) queues whatever it likes on the view's stream.  in, out and
//              extra[] name buffers (-1 for none; out is required and decides the rows covered);
//              call_flags as above; partial_floats: floats per sequence and chunk it wants at
//              view->partial.  On a cache group with a window it sees steps of up to 256 tokens a
//              sequence (what the group's ring takes in at once): a longer one is refused, and the
//              caller cuts the prompt into continuation steps.
typedef struct {
    int32_t kind, rows;
    int32_t in, out;
    const void* weight;
    int32_t weight_dt, n, k, epilogue;
    float eps;
    const float* in_norm_weight;
    float in_norm_eps;
    int32_t in_norm_x;
    const float* out_norm_weight;
    float out_norm_eps;
    int32_t out_norm_when;
    int32_t n_heads, n_kv_heads, head_dim, window;
    float scale;
    const float* cos_table;
    const float* sin_table;
    int32_t rope_style, table_positions;
    int32_t kv_group, kv_entry, kv_writes, q_buffer;
    picolm_call_fn call;
    void* call_user;
    int32_t call_flags;
    int32_t state_group, state_entry;
    int32_t extra[4];
    int32_t tile_rows, partial_floats;
} picolm_op;

// Keys and values of `n_entries` layer calls that need the same kind of cache.  window > 0: the
// group keeps the last `window` keys of a sequence in a ring of pages (enough for a window and a
// prefill chunk of 256 tokens); 0: all keys.  v_head_dim: the size of a value where it is not that
// of a key (0: the same); the ATTENTION operation takes one size for both, a called operation any.
typedef struct {
    int32_t n_entries, n_kv_heads, head_dim, window, v_head_dim;
} picolm_kv_group;

// Fixed-size state per sequence for `n_entries` layer calls, zeroed when a slot is given out.
typedef struct {
    int32_t n_entries;
    int64_t bytes_per_slot;
} picolm_state_group;

typedef struct {
    int32_t dtype;           // PICOLM_BF16: serving precision; PICOLM_F32: true 32-bit
    int32_t vocab_size;
    const picolm_op* ops;
    int32_t n_ops;
    const picolm_buffer* buffers;
    int32_t n_buffers;
    int32_t logits_buffer;   // float rows [vocab_size], PICOLM_ROWS_WANTED
    const picolm_kv_group* kv_groups;
    int32_t n_kv_groups;
    const picolm_state_group* state_groups;
    int32_t n_state_groups;
} picolm_program;

#define PICOLM_ENGINE_NO_GRAPHS 1    // launch every decode step's kernels one by one
#define PICOLM_ENGINE_HOST_ONLY 2    // books and index arrays only, no device memory: steps plan but do not run
#define PICOLM_ENGINE_TIME_OPS 4     // an event before and after every operation (decode steps are then launched, not replayed)

typedef struct picolm_engine picolm_engine;

// max_tokens: the most tokens live sequences hold together, each sequence's count rounded up to
// pages of 64; max_seq_len: the longest one sequence may get; n_slots: 0 gives one per page.
// The program is copied; the weights and tables it points to must outlive the engine.
int picolm_engine_create(const picolm_program* program, int64_t max_tokens, int32_t max_seq_len, int32_t n_slots,
                         int32_t flags, picolm_engine** out);
void picolm_engine_destroy(picolm_engine* e);

int picolm_engine_slot_alloc(picolm_engine* e, int32_t* slot, hipStream_t stream);
int picolm_engine_slot_free(picolm_engine* e, int32_t slot);
int picolm_engine_slot_length(picolm_engine* e, int32_t slot);      // tokens the slot holds, negative: not live

// One step.  Sequence i lives in slots[i] and brings n_new[i] >= 1 tokens, packed in `tokens`
// (host memory) in the order of the sequences; they are appended at the slot's length.  The
// sequences of a step either all bring prompts (any lengths) or one token each.  want_counts[i]
// indices into sequence i's new tokens are listed, packed, in `want`; want_counts null: each
// sequence's last token.  *logits: float [*n_rows][vocab] in device memory that the engine owns,
// valid until the next step of this engine, in the order of the sequences and of `want`.  A
// refused step (PICOLM_ERR_STEP, PICOLM_ERR_CACHE_FULL) leaves every sequence where it was.
int picolm_engine_step(picolm_engine* e, int32_t n_seq, const int32_t* slots, const int32_t* n_new,
                       const int32_t* tokens, const int32_t* want_counts, const int32_t* want, float** logits,
                       int32_t* n_rows, hipStream_t stream);
// One more token for each sequence, the tokens lying in device memory (what a sampling kernel
// wrote, or will have written when the step runs); they must lie inside the vocabulary.
int picolm_engine_step_device_tokens(picolm_engine* e, int32_t n_seq, const int32_t* slots, const int32_t* tokens_dev,
                                     float** logits, hipStream_t stream);

// Sampling options with picolm's meanings (picolm/sampler.h:6-12): temperature <= 0 is greedy,
// top_k 0 is off, top_p 1 and min_p 0 are off, seed 0 becomes 42.
typedef struct {
    float temperature;
    int32_t top_k;
    float top_p, min_p;
    uint64_t seed;
} picolm_sampling;

// The generation loop (picolm/picolm.c:1502-1610) over batches of unequal prompts: prompts of a
// batch in one step, then one token each; a sequence ends with a stop token (recorded), after
// max_new tokens, or at the cache's capacity, leaves the batch and gives its slot back; batches of
// up to batch_size requests follow each other until all are done.  prompts: packed token ids,
// prompt_lens[i] >= 1 each.  out_tokens: [n_prompts][max_new]; out_counts[i] tokens were made;
// out_finish[i]: 1 stop token, 2 length, 3 capacity.  Decoding runs one step ahead of the host: a
// step is queued before the tokens of the step before it have been read, so the GPU does not stand
// still while the host decides (a sequence that a stop token ends has then been stepped once more;
// that step's token is dropped).  Prompts
// of a batch that together exceed the step's token budget (16,384 unless set otherwise; it sizes
// the workspace) go in as several steps, each appending to what the slots hold.
int picolm_engine_set_prefill_step_tokens(picolm_engine* e, int32_t tokens);
int picolm_engine_generate(picolm_engine* e, int32_t n_prompts, const int32_t* prompts, const int32_t* prompt_lens,
                           int32_t max_new, const picolm_sampling* sampling, const int32_t* stop_ids, int32_t n_stop,
                           int32_t batch_size, int32_t* out_tokens, int32_t* out_counts, int32_t* out_finish,
                           hipStream_t stream);

// With PICOLM_ENGINE_TIME_OPS: the GPU time in milliseconds since the last call, summed by class
// of operation: ms[0] embedding and norms of their own, ms[1] the layers' products (with the norms
// and partial sums that belong to them), ms[2] the head's product, ms[3] attention (with rotation
// and the cache write).  Waits for the GPU.  picolm prints such figures for its layers itself
// (picolm/picolm.c:305-317).
int picolm_engine_op_times(picolm_engine* e, double* ms);

// ---- what the engine holds, for bindings and tests ---------------------------------------------
// what: 0 max_seq_len, 1 n_slots, 2 free slots, 3 free tokens (pages free in the tightest group
// times 64; 2^40 for a model without cache groups), 4 recorded decode steps, 5 pages of a
// sequence's table row, 6 bytes of device memory held, 7 the counter that moves when a slot or
// page changes hands, 8 the most tokens a sequence may bring in one step (0: any number; 256
// where a called operation uses a group with a window), 9 bytes of keys, values and state
int64_t picolm_engine_info(picolm_engine* e, int32_t what);
// keys [n_pages][G][64][d] and values [n_pages][G][d][64] of one cache entry (device memory)
int picolm_engine_kv_entry(picolm_engine* e, int32_t group, int32_t entry, void** k, void** v, int64_t* n_pages);
// state [n_slots][bytes_per_slot] of one entry (device memory)
int picolm_engine_state_entry(picolm_engine* e, int32_t group, int32_t entry, void** state, int64_t* bytes_per_slot);
// the pages a slot holds in a group, in logical order; returns their number (negative: error)
int picolm_engine_slot_pages(picolm_engine* e, int32_t group, int32_t slot, int32_t* pages, int32_t capacity);
int picolm_engine_free_pages(picolm_engine* e, int32_t group);
// One of the index arrays of the step planned last, by name, from the host's copy: "seq_slot",
// "seq_pos0", "seq_nnew", "cu_seqlens", "tok_pos", "tok_seq", "tokens", "want_rows",
// "write_pages.<group>", "chunks.<group>" (the decode work list with its header),
// "tiles.<rows>.seq", "tiles.<rows>.q0", and of slice c of a prefill step for the groups that keep a
// ring "window_chunk.<c>.seq_slot", ".seq_pos0", ".seq_nnew", ".first_row", ".rows", ".tiles.<rows>.seq",
// ".tiles.<rows>.q0".  Returns the number of ints (negative: no such array).
int picolm_engine_step_array(picolm_engine* e, const char* name, int32_t* out, int32_t capacity);

#ifdef __cplusplus
}
#endif
