/* A client of the library's C API written in C: it builds the launch program of a two-layer Llama
 * by hand (the operations of csrc/engine.h, nothing of the Python parts), makes the engine, steps
 * a batch of two unequal prompts and three single tokens each, lets the library's own loop
 * generate greedily, and holds every row of logits against a plain forward pass over whole
 * sequences written below in double precision (the formulas of picolm/model_core.c:1785-2220:
 * embedding, RMSNorm, q/k/v, pairwise rotation, attention over keys t <= pos, output product and
 * residual, SwiGLU, final norm and head).
 *
 *   tiny_llama_c f32|bf16      exit 0 and "ok ..." when everything agrees
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "engine.h"
#include "api.h"

enum { D = 64, H = 4, G = 2, HD = 16, F = 96, V = 101, L = 2, MAXPOS = 128 };
#define EPS 1e-5f
#define THETA 10000.0

#define CHECK_HIP(call)                                                               \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                       \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                \
            exit(2);                                                                  \
        }                                                                             \
    } while (0)
#define CHECK_LIB(call)                                                               \
    do {                                                                              \
        int rc_ = (call);                                                             \
        if (rc_ != 0) {                                                               \
            fprintf(stderr, "%s: %d: %s\n", #call, rc_, picolm_last_error());         \
            exit(2);                                                                  \
        }                                                                             \
    } while (0)

/* ---- weights: values that bfloat16 holds exactly, from a small generator ---------------------- */
static uint32_t rng_state = 12345u;
static float next_uniform(void) { /* in (-1, 1) */
    rng_state = rng_state * 1664525u + 1013904223u;
    return ((float)(rng_state >> 8) / 8388608.0f) - 1.0f;
}
static uint16_t to_bf16_bits(float f) { /* round to nearest even */
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16_bits(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static float* random_matrix(int rows, int cols, float spread) {
    float* w = malloc(sizeof(float) * rows * cols);
    for (int i = 0; i < rows * cols; ++i) w[i] = from_bf16_bits(to_bf16_bits(next_uniform() * spread));
    return w;
}
/* a matrix on the device in the engine's weight type */
static void* upload_matrix(const float* w, size_t n, int bf16) {
    void* dev = NULL;
    if (bf16) {
        uint16_t* h = malloc(2 * n);
        for (size_t i = 0; i < n; ++i) h[i] = to_bf16_bits(w[i]);
        CHECK_HIP(hipMalloc(&dev, 2 * n));
        CHECK_HIP(hipMemcpy(dev, h, 2 * n, hipMemcpyHostToDevice));
        free(h);
    } else {
        CHECK_HIP(hipMalloc(&dev, 4 * n));
        CHECK_HIP(hipMemcpy(dev, w, 4 * n, hipMemcpyHostToDevice));
    }
    return dev;
}
static float* upload_floats(const float* w, size_t n) { return (float*)upload_matrix(w, n, 0); }

typedef struct {
    float *norm1, *wq, *wk, *wv, *wo, *norm2, *wg, *wu, *wd;
} layer_weights;
static float *emb, *final_norm, *head;
static layer_weights layers[L];

/* ---- the plain forward pass: whole sequence, no cache, double precision ---------------------- */
static void rmsnorm(const double* x, const float* w, double* out, int n) {
    double ss = 0.0;
    for (int i = 0; i < n; ++i) ss += x[i] * x[i];
    const double r = 1.0 / sqrt(ss / n + (double)EPS);
    for (int i = 0; i < n; ++i) out[i] = x[i] * r * w[i];
}
static void matvec(const float* w, const double* x, double* y, int rows, int cols) {
    for (int r = 0; r < rows; ++r) {
        double s = 0.0;
        for (int c = 0; c < cols; ++c) s += (double)w[r * cols + c] * x[c];
        y[r] = s;
    }
}
static void rotate(double* v, int pos) { /* pairs (2i, 2i+1), angle pos / theta^(2i/d) */
    for (int i = 0; i < HD / 2; ++i) {
        const double angle = (double)pos / pow(THETA, 2.0 * i / HD);
        const double c = cos(angle), s = sin(angle), a = v[2 * i], b = v[2 * i + 1];
        v[2 * i] = a * c - b * s;
        v[2 * i + 1] = a * s + b * c;
    }
}
/* logits [T][V] of the sequence `tokens` */
static double* plain_logits(const int32_t* tokens, int T) {
    double* x = malloc(sizeof(double) * T * D);
    double* q = malloc(sizeof(double) * T * H * HD);
    double* k = malloc(sizeof(double) * T * G * HD);
    double* v = malloc(sizeof(double) * T * G * HD);
    double h[D], att[H * HD], o[D], gate[F], up[F], scores[MAXPOS];
    for (int t = 0; t < T; ++t)
        for (int i = 0; i < D; ++i) x[t * D + i] = emb[tokens[t] * D + i];
    for (int l = 0; l < L; ++l) {
        const layer_weights* w = &layers[l];
        for (int t = 0; t < T; ++t) {
            rmsnorm(x + t * D, w->norm1, h, D);
            matvec(w->wq, h, q + t * H * HD, H * HD, D);
            matvec(w->wk, h, k + t * G * HD, G * HD, D);
            matvec(w->wv, h, v + t * G * HD, G * HD, D);
            for (int i = 0; i < H; ++i) rotate(q + (t * H + i) * HD, t);
            for (int i = 0; i < G; ++i) rotate(k + (t * G + i) * HD, t);
        }
        for (int t = 0; t < T; ++t) {
            for (int i = 0; i < H; ++i) {
                const int g = i / (H / G);
                double top = -1e300, sum = 0.0;
                for (int u = 0; u <= t; ++u) {
                    double s = 0.0;
                    for (int j = 0; j < HD; ++j) s += q[(t * H + i) * HD + j] * k[(u * G + g) * HD + j];
                    scores[u] = s / sqrt((double)HD);
                    if (scores[u] > top) top = scores[u];
                }
                for (int u = 0; u <= t; ++u) {
                    scores[u] = exp(scores[u] - top);
                    sum += scores[u];
                }
                for (int j = 0; j < HD; ++j) {
                    double a = 0.0;
                    for (int u = 0; u <= t; ++u) a += scores[u] * v[(u * G + g) * HD + j];
                    att[i * HD + j] = a / sum;
                }
            }
            matvec(w->wo, att, o, D, H * HD);
            for (int i = 0; i < D; ++i) x[t * D + i] += o[i];
            rmsnorm(x + t * D, w->norm2, h, D);
            matvec(w->wg, h, gate, F, D);
            matvec(w->wu, h, up, F, D);
            for (int i = 0; i < F; ++i) gate[i] = gate[i] / (1.0 + exp(-gate[i])) * up[i];
            matvec(w->wd, gate, o, D, F);
            for (int i = 0; i < D; ++i) x[t * D + i] += o[i];
        }
    }
    double* logits = malloc(sizeof(double) * T * V);
    for (int t = 0; t < T; ++t) {
        rmsnorm(x + t * D, final_norm, h, D);
        matvec(head, h, logits + t * V, V, D);
    }
    free(x), free(q), free(k), free(v);
    return logits;
}
static int argmax(const double* row) {
    int best = 0;
    for (int i = 1; i < V; ++i)
        if (row[i] > row[best]) best = i;
    return best;
}

/* ---- the program ------------------------------------------------------------------------------ */
enum { B_X, B_H, B_QKV, B_Q, B_ATT, B_ACT, B_HF, B_LOGITS, N_BUFFERS };

int main(int argc, char** argv) {
    const int bf16 = argc > 1 && strcmp(argv[1], "bf16") == 0;
    const int dtype = bf16 ? PICOLM_BF16 : PICOLM_F32, item = bf16 ? 2 : 4;
    /* the bound of the Python tests (tests/tiny.py): this share of the largest logit, of 1 if that is smaller */
    const double share = bf16 ? 2e-2 : 2e-5;
    double largest = 1.0;
    CHECK_LIB(picolm_device_check());

    emb = random_matrix(V, D, 1.0f);
    head = random_matrix(V, D, 0.3f);
    final_norm = random_matrix(1, D, 0.2f);
    for (int i = 0; i < D; ++i) final_norm[i] += 1.0f;
    void* emb_dev = upload_matrix(emb, (size_t)V * D, bf16);
    void* head_dev = upload_matrix(head, (size_t)V * D, bf16);
    float* final_dev = upload_floats(final_norm, D);

    /* rotation tables [MAXPOS][HD / 2] */
    float* cos_t = malloc(sizeof(float) * MAXPOS * HD / 2);
    float* sin_t = malloc(sizeof(float) * MAXPOS * HD / 2);
    for (int p = 0; p < MAXPOS; ++p)
        for (int i = 0; i < HD / 2; ++i) {
            const double angle = (double)p / pow(THETA, 2.0 * i / HD);
            cos_t[p * (HD / 2) + i] = (float)cos(angle);
            sin_t[p * (HD / 2) + i] = (float)sin(angle);
        }
    float* cos_dev = upload_floats(cos_t, (size_t)MAXPOS * HD / 2);
    float* sin_dev = upload_floats(sin_t, (size_t)MAXPOS * HD / 2);

    picolm_buffer buffers[N_BUFFERS] = {
        [B_X] = {4 * D, PICOLM_ROWS_STEP, PICOLM_F32},
        [B_H] = {item * D, PICOLM_ROWS_STEP, dtype},
        [B_QKV] = {4 * (H + 2 * G) * HD, PICOLM_ROWS_STEP, PICOLM_F32},
        [B_Q] = {item * H * HD, PICOLM_ROWS_STEP, dtype},
        [B_ATT] = {item * H * HD, PICOLM_ROWS_STEP, dtype},
        [B_ACT] = {item * F, PICOLM_ROWS_STEP, dtype},
        [B_HF] = {item * D, PICOLM_ROWS_WANTED, dtype},
        [B_LOGITS] = {4 * V, PICOLM_ROWS_WANTED, PICOLM_F32},
    };
    picolm_op ops[2 + 5 * L];
    memset(ops, 0, sizeof(ops));
    int n_ops = 0;
    picolm_op* o = &ops[n_ops++];
    o->kind = PICOLM_OP_EMBED, o->rows = PICOLM_ROWS_STEP, o->in = -1, o->out = B_X;
    o->weight = emb_dev, o->weight_dt = dtype, o->n = V, o->k = D;
    const float* next_norm[L + 1];
    for (int l = 0; l < L; ++l) {
        layer_weights* w = &layers[l];
        w->norm1 = random_matrix(1, D, 0.2f), w->norm2 = random_matrix(1, D, 0.2f);
        for (int i = 0; i < D; ++i) w->norm1[i] += 1.0f, w->norm2[i] += 1.0f;
        w->wq = random_matrix(H * HD, D, 0.2f), w->wk = random_matrix(G * HD, D, 0.2f), w->wv = random_matrix(G * HD, D, 0.2f);
        w->wo = random_matrix(D, H * HD, 0.2f);
        w->wg = random_matrix(F, D, 0.2f), w->wu = random_matrix(F, D, 0.2f), w->wd = random_matrix(D, F, 0.2f);
        /* q, k, v stacked along the output rows; gate and up with their rows taking turns */
        float* qkv = malloc(sizeof(float) * (H + 2 * G) * HD * D);
        memcpy(qkv, w->wq, sizeof(float) * H * HD * D);
        memcpy(qkv + H * HD * D, w->wk, sizeof(float) * G * HD * D);
        memcpy(qkv + (H + G) * HD * D, w->wv, sizeof(float) * G * HD * D);
        float* gu = malloc(sizeof(float) * 2 * F * D);
        for (int r = 0; r < F; ++r) {
            memcpy(gu + (2 * r) * D, w->wg + r * D, sizeof(float) * D);
            memcpy(gu + (2 * r + 1) * D, w->wu + r * D, sizeof(float) * D);
        }
        void* qkv_dev = upload_matrix(qkv, (size_t)(H + 2 * G) * HD * D, bf16);
        void* wo_dev = upload_matrix(w->wo, (size_t)D * H * HD, bf16);
        void* gu_dev = upload_matrix(gu, (size_t)2 * F * D, bf16);
        void* wd_dev = upload_matrix(w->wd, (size_t)D * F, bf16);
        float* n1_dev = upload_floats(w->norm1, D);
        float* n2_dev = upload_floats(w->norm2, D);
        next_norm[l] = n1_dev;
        free(qkv), free(gu);

        o = &ops[n_ops++]; /* q, k, v = W rmsnorm(x) */
        o->kind = PICOLM_OP_LINEAR, o->rows = PICOLM_ROWS_STEP, o->in = B_H, o->out = B_QKV;
        o->weight = qkv_dev, o->weight_dt = dtype, o->n = (H + 2 * G) * HD, o->k = D, o->epilogue = 0;
        o->in_norm_weight = n1_dev, o->in_norm_eps = EPS, o->in_norm_x = B_X;
        o = &ops[n_ops++]; /* rotation, cache write, attention */
        o->kind = PICOLM_OP_ATTENTION, o->rows = PICOLM_ROWS_STEP, o->in = B_QKV, o->out = B_ATT, o->q_buffer = B_Q;
        o->n_heads = H, o->n_kv_heads = G, o->head_dim = HD, o->window = 0, o->scale = 1.0f / sqrtf((float)HD);
        o->cos_table = cos_dev, o->sin_table = sin_dev, o->rope_style = 0, o->table_positions = MAXPOS;
        o->kv_group = 0, o->kv_entry = l, o->kv_writes = 1;
        o = &ops[n_ops++]; /* x += Wo attention, and the norm that follows may be prepared */
        o->kind = PICOLM_OP_LINEAR, o->rows = PICOLM_ROWS_STEP, o->in = B_ATT, o->out = B_X;
        o->weight = wo_dev, o->weight_dt = dtype, o->n = D, o->k = H * HD, o->epilogue = 1;
        o->out_norm_weight = n2_dev, o->out_norm_eps = EPS;
        o = &ops[n_ops++]; /* silu(gate) * up of rmsnorm(x) */
        o->kind = PICOLM_OP_LINEAR, o->rows = PICOLM_ROWS_STEP, o->in = B_H, o->out = B_ACT;
        o->weight = gu_dev, o->weight_dt = dtype, o->n = 2 * F, o->k = D, o->epilogue = 2;
        o->in_norm_weight = n2_dev, o->in_norm_eps = EPS, o->in_norm_x = B_X;
        o = &ops[n_ops++]; /* x += Wd act */
        o->kind = PICOLM_OP_LINEAR, o->rows = PICOLM_ROWS_STEP, o->in = B_ACT, o->out = B_X;
        o->weight = wd_dev, o->weight_dt = dtype, o->n = D, o->k = F, o->epilogue = 1;
    }
    next_norm[L] = final_dev;
    for (int l = 0; l < L; ++l) { /* each layer's last product knows the norm that meets x next */
        picolm_op* down = &ops[1 + 5 * l + 4];
        down->out_norm_weight = next_norm[l + 1], down->out_norm_eps = EPS, down->out_norm_when = l == L - 1;
    }
    o = &ops[n_ops++]; /* the head over the wanted rows of rmsnorm(x) */
    o->kind = PICOLM_OP_LINEAR, o->rows = PICOLM_ROWS_WANTED, o->in = B_HF, o->out = B_LOGITS;
    o->weight = head_dev, o->weight_dt = dtype, o->n = V, o->k = D, o->epilogue = 0;
    o->in_norm_weight = final_dev, o->in_norm_eps = EPS, o->in_norm_x = B_X;

    picolm_kv_group group = {L, G, HD, 0, 0};
    picolm_program program = {dtype, V, ops, n_ops, buffers, N_BUFFERS, B_LOGITS, &group, 1, NULL, 0};
    picolm_engine* engine = NULL;
    CHECK_LIB(picolm_engine_create(&program, 64 * 8, MAXPOS, 4, 0, &engine));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));

    /* two prompts of unequal lengths in one step, then three tokens each */
    enum { NA = 9, NB = 5, MORE = 3 };
    int32_t seq_a[NA + MORE], seq_b[NB + MORE];
    for (int i = 0; i < NA; ++i) seq_a[i] = (7 * i + 3) % V;
    for (int i = 0; i < NB; ++i) seq_b[i] = (11 * i + 5) % V;
    int32_t slots[2];
    CHECK_LIB(picolm_engine_slot_alloc(engine, &slots[0], stream));
    CHECK_LIB(picolm_engine_slot_alloc(engine, &slots[1], stream));
    int32_t n_new[2] = {NA, NB}, packed[NA + NB], want_counts[2] = {2, 1}, want[3] = {0, NA - 1, NB - 1};
    memcpy(packed, seq_a, sizeof(int32_t) * NA);
    memcpy(packed + NA, seq_b, sizeof(int32_t) * NB);
    float* logits_dev = NULL;
    int32_t n_rows = 0;
    float got[3 * V];
    double worst = 0.0;
    CHECK_LIB(picolm_engine_step(engine, 2, slots, n_new, packed, want_counts, want, &logits_dev, &n_rows, stream));
    if (n_rows != 3) return fprintf(stderr, "the prompt step gave %d rows\n", n_rows), 1;
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(got, logits_dev, sizeof(float) * 3 * V, hipMemcpyDeviceToHost));
    {
        double* ra = plain_logits(seq_a, NA);
        double* rb = plain_logits(seq_b, NB);
        const double* rows[3] = {ra, ra + (NA - 1) * V, rb + (NB - 1) * V};
        for (int r = 0; r < 3; ++r)
            for (int i = 0; i < V; ++i) {
                worst = fmax(worst, fabs(got[r * V + i] - rows[r][i]));
                largest = fmax(largest, fabs(rows[r][i]));
            }
        seq_a[NA] = argmax(ra + (NA - 1) * V);
        seq_b[NB] = argmax(rb + (NB - 1) * V);
        free(ra), free(rb);
    }
    for (int step = 0; step < MORE; ++step) {
        int32_t ones[2] = {1, 1}, toks[2] = {seq_a[NA + step], seq_b[NB + step]};
        CHECK_LIB(picolm_engine_step(engine, 2, slots, ones, toks, NULL, NULL, &logits_dev, &n_rows, stream));
        CHECK_HIP(hipStreamSynchronize(stream));
        CHECK_HIP(hipMemcpy(got, logits_dev, sizeof(float) * 2 * V, hipMemcpyDeviceToHost));
        double* ra = plain_logits(seq_a, NA + step + 1);
        double* rb = plain_logits(seq_b, NB + step + 1);
        for (int i = 0; i < V; ++i) {
            worst = fmax(worst, fabs(got[i] - ra[(NA + step) * V + i]));
            worst = fmax(worst, fabs(got[V + i] - rb[(NB + step) * V + i]));
            largest = fmax(largest, fmax(fabs(ra[(NA + step) * V + i]), fabs(rb[(NB + step) * V + i])));
        }
        if (step + 1 < MORE) {
            seq_a[NA + step + 1] = argmax(ra + (NA + step) * V);
            seq_b[NB + step + 1] = argmax(rb + (NB + step) * V);
        }
        free(ra), free(rb);
    }
    if (picolm_engine_slot_length(engine, slots[0]) != NA + MORE || picolm_engine_slot_length(engine, slots[1]) != NB + MORE)
        return fprintf(stderr, "the slots hold %d and %d tokens\n", picolm_engine_slot_length(engine, slots[0]),
                       picolm_engine_slot_length(engine, slots[1])), 1;
    CHECK_LIB(picolm_engine_slot_free(engine, slots[0]));
    CHECK_LIB(picolm_engine_slot_free(engine, slots[1]));
    const double tolerance = share * largest;
    if (!(worst <= tolerance)) return fprintf(stderr, "logits differ from the plain forward pass by %g (allowed %g)\n", worst, tolerance), 1;

    /* the library's own loop, greedy: the tokens of the plain forward pass (ties aside: the margins are printed) */
    enum { NEW = 4 };
    int32_t prompt_lens[2] = {NA, NB}, out_tokens[2 * NEW], out_counts[2], out_finish[2];
    picolm_sampling greedy = {0.0f, 0, 1.0f, 0.0f, 0};
    CHECK_LIB(picolm_engine_generate(engine, 2, packed, prompt_lens, NEW, &greedy, NULL, 0, 2, out_tokens, out_counts, out_finish, stream));
    for (int r = 0; r < 2; ++r) {
        int32_t seq[NA + NEW];
        const int n0 = r == 0 ? NA : NB;
        memcpy(seq, r == 0 ? seq_a : seq_b, sizeof(int32_t) * n0);
        if (out_counts[r] != NEW || out_finish[r] != 2) return fprintf(stderr, "request %d made %d tokens, finish %d\n", r, out_counts[r], out_finish[r]), 1;
        for (int j = 0; j < NEW; ++j) {
            double* ref = plain_logits(seq, n0 + j);
            const double* row = ref + (n0 + j - 1) * V;
            const int tok = out_tokens[r * NEW + j];
            if (row[tok] < row[argmax(row)] - 2.0 * tolerance)
                return fprintf(stderr, "request %d token %d: %d where the plain pass has %d\n", r, j, tok, argmax(row)), 1;
            seq[n0 + j] = tok;
            free(ref);
        }
    }
    picolm_engine_destroy(engine);
    printf("ok %s: worst difference of the logits %.3g (allowed %g)\n", bf16 ? "bf16" : "f32", worst, tolerance);
    return 0;
}
