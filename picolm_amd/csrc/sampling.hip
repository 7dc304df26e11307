// Token choice on the GPU, one workgroup per row of logits.
//
// Greedy: the first maximum (picolm/sampler.c:50-55, strict '>' keeps the lowest index).
// Otherwise picolm's pipeline (picolm/sampler.c:58-121): softmax of the raw logits, order by
// probability descending, keep the first top_k, cut where the cumulative probability reaches
// top_p, drop what is below min_p times the largest, raise to 1/T and renormalise, draw with
// xorshift64: the first position whose running sum exceeds r.
//
// Nothing is sorted here.  Every stage of that pipeline keeps a prefix of the descending
// order, and a prefix is named by its last element: (key, index) with key a monotone 32-bit
// image of the logit and equal logits ordered by ascending token id.  The element where a
// running sum crosses a target is found by descending a 256-way histogram of a 24-bit linear
// quantisation of the logits (weights summed per bucket in double), then ordering the few
// elements of the final bucket exactly.  Sums are double so that the order of addition
// cannot change a decision in practice.
#include "common.h"
#include "api.h"

#define SM_THREADS 1024
#define SM_LIST 1024
#define SM_WAVES (SM_THREADS / WAVE)

// Stage 1: a row is cut into slices of ARGMAX_SLICE values, one workgroup each, which leave their
// (maximum, lowest index of it) in `part`; stage 2 picks among a row's slices.  A row of 128k
// logits is 32 workgroups instead of one.
#define ARGMAX_SLICE 4096
#define ARGMAX_THREADS 256

__device__ __forceinline__ void argmax_merge(float& best, int& best_i, float ov, int oi) {
    if (oi != 0x7fffffff && (best_i == 0x7fffffff || ov > best || (ov == best && oi < best_i))) {
        best = ov;
        best_i = oi;
    }
}

__device__ __forceinline__ void argmax_block(float& best, int& best_i, float* sv, int* si) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(best_i, o, WAVE);
        argmax_merge(best, best_i, ov, oi);
    }
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (lane == 0) {
        sv[wave] = best;
        si[wave] = best_i;
    }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < (int)blockDim.x / WAVE; ++w) argmax_merge(best, best_i, sv[w], si[w]);
}

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_slice_kernel(const float* __restrict__ logits,
                                                                      float* __restrict__ part_v,
                                                                      int32_t* __restrict__ part_i, int V,
                                                                      int64_t ld, int n_slices) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (int64_t)blockIdx.y * ld;
    const int lo = blockIdx.x * ARGMAX_SLICE, hi = min(V, lo + ARGMAX_SLICE);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += ARGMAX_THREADS) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) {      // the first element seen, or strictly greater
            best = v;
            best_i = i;
        }
    }
    argmax_block(best, best_i, sv, si);
    if (threadIdx.x == 0) {
        part_v[(size_t)blockIdx.y * n_slices + blockIdx.x] = best;
        part_i[(size_t)blockIdx.y * n_slices + blockIdx.x] = best_i;
    }
}

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_pick_kernel(const float* __restrict__ part_v,
                                                                     const int32_t* __restrict__ part_i,
                                                                     int32_t* __restrict__ out, int n_slices) {
    __shared__ float sv[16];
    __shared__ int si[16];
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int s = threadIdx.x; s < n_slices; s += ARGMAX_THREADS)
        argmax_merge(best, best_i, part_v[(size_t)blockIdx.x * n_slices + s], part_i[(size_t)blockIdx.x * n_slices + s]);
    argmax_block(best, best_i, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
}

extern "C" int picolm_argmax_scratch_floats(int n_rows, int V) { return 2 * n_rows * ceil_div(V, ARGMAX_SLICE); }

// `scratch`: picolm_argmax_scratch_floats(n_rows, V) floats of device memory
extern "C" int picolm_argmax(const float* logits, int32_t* out, int n_rows, int V, int64_t ld, float* scratch,
                             hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d ld=%lld", n_rows, V,
                   (long long)ld);
    PICOLM_REQUIRE(scratch != nullptr, "argmax: needs its scratch buffer");
    PICOLM_REQUIRE(n_rows <= 65535, "argmax: %d rows exceed the grid", n_rows);
    if (n_rows == 0) return 0;
    const int n_slices = ceil_div(V, ARGMAX_SLICE);
    float* part_v = scratch;
    int32_t* part_i = (int32_t*)(scratch + (size_t)n_rows * n_slices);
    argmax_slice_kernel<<<dim3(n_slices, n_rows), dim3(ARGMAX_THREADS), 0, stream>>>(logits, part_v, part_i, V, ld, n_slices);
    PICOLM_LAUNCH_CHECK("argmax");
    argmax_pick_kernel<<<dim3(n_rows), dim3(ARGMAX_THREADS), 0, stream>>>(part_v, part_i, out, n_slices);
    PICOLM_LAUNCH_CHECK("argmax");
    return 0;
}

// ---------------------------------------------------------------------------------------------
struct Prefix {       // element (k, i) belongs iff k > key || (k == key && i <= idx)
    uint32_t key;
    int idx;
};
#define PREFIX_ALL (Prefix{0u, 0x7fffffff})

__device__ __forceinline__ uint32_t order_key(float l) {
    if (l == 0.0f) l = 0.0f;                       // -0 and +0 are one value
    const uint32_t u = __float_as_uint(l);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ bool in_prefix(uint32_t k, int i, Prefix p) {
    return k > p.key || (k == p.key && i <= p.idx);
}

struct RowInfo {
    const float* row;
    int V;
    float lmin;
    double lmax;
    double qscale;
    double inv_t;
};
__device__ __forceinline__ uint32_t quant24(const RowInfo& r, float l) {
    const double s = ((double)l - (double)r.lmin) * r.qscale;
    return s >= 16777215.0 ? 16777215u : (uint32_t)s;
}
// mode 0: exp(l - max); mode 1: exp((l - max)/T); mode 2: nothing is weighed, elements are counted
__device__ __forceinline__ double weight_of(const RowInfo& r, float l, int mode) {
    if (mode == 2) return 0.0;
    const double x = (double)l - r.lmax;
    return exp(mode == 1 ? x * r.inv_t : x);
}

struct SampleShared {
    double hist_w[256];
    unsigned hist_c[256];
    double red_d[SM_WAVES];
    unsigned red_u[SM_WAVES];
    int list_idx[SM_LIST];
    uint32_t list_key[SM_LIST];
    int sorted_idx[SM_LIST];
    uint32_t sorted_key[SM_LIST];
    double sorted_w[SM_LIST];
    unsigned n_list;
    int chosen;
    double base_w;
    unsigned base_c;
    Prefix res;
    unsigned res_count;
    int found;
    unsigned bcast_u;
    int bcast_i;
};

__device__ double block_sum_f64(double v, SampleShared& sm) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    __syncthreads();
    if (threadIdx.x % WAVE == 0) sm.red_d[threadIdx.x / WAVE] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < SM_WAVES; ++i) t += sm.red_d[i];
    return t;
}
__device__ unsigned block_max_u32(unsigned v, SampleShared& sm) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v = max(v, (unsigned)__shfl_xor((int)v, o, WAVE));
    __syncthreads();
    if (threadIdx.x % WAVE == 0) sm.red_u[threadIdx.x / WAVE] = v;
    __syncthreads();
    unsigned t = 0;
    for (int i = 0; i < SM_WAVES; ++i) t = max(t, sm.red_u[i]);
    return t;
}
__device__ unsigned block_min_u32(unsigned v, SampleShared& sm) { return ~block_max_u32(~v, sm); }
__device__ unsigned block_sum_u32(unsigned v, SampleShared& sm) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += (unsigned)__shfl_xor((int)v, o, WAVE);
    __syncthreads();
    if (threadIdx.x % WAVE == 0) sm.red_u[threadIdx.x / WAVE] = v;
    __syncthreads();
    unsigned t = 0;
    for (int i = 0; i < SM_WAVES; ++i) t += sm.red_u[i];
    return t;
}

// Index of the t-th (1-based) element, in ascending index order, with key == k inside `within`.
__device__ int nth_tie(const RowInfo& r, uint32_t k, Prefix within, unsigned t, SampleShared& sm) {
    const int chunk = (r.V + SM_THREADS - 1) / SM_THREADS;
    const int b = threadIdx.x * chunk, e = min(r.V, b + chunk);
    unsigned c = 0;
    for (int i = b; i < e; ++i) c += (order_key(r.row[i]) == k && in_prefix(k, i, within)) ? 1u : 0u;
    __syncthreads();
    sm.list_idx[threadIdx.x] = (int)c;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned cum = 0;
        int owner = -1;
        unsigned local = 0;
        for (int j = 0; j < SM_THREADS; ++j) {
            if (cum + (unsigned)sm.list_idx[j] >= t) {
                owner = j;
                local = t - cum;
                break;
            }
            cum += (unsigned)sm.list_idx[j];
        }
        sm.bcast_i = owner;
        sm.bcast_u = local;
    }
    __syncthreads();
    const int owner = sm.bcast_i;
    const unsigned local = sm.bcast_u;
    __syncthreads();
    if (owner == (int)threadIdx.x) {
        unsigned seen = 0;
        int found = e - 1;
        for (int i = b; i < e; ++i)
            if (order_key(r.row[i]) == k && in_prefix(k, i, within) && ++seen == local) {
                found = i;
                break;
            }
        sm.bcast_i = found;
    }
    __syncthreads();
    const int res = owner < 0 ? 0x7fffffff : sm.bcast_i;   // fewer ties than asked: all of them
    __syncthreads();
    return res;
}

// Walk the elements of `within` in descending order, summing weights; stop at the first
// element where the sum crosses `target` (strict: sum > target, else sum >= target) or the
// count reaches `limit`.  Leaves in sm.res the prefix ending at that element, in sm.res_count
// its size, in sm.found whether a crossing happened (otherwise the prefix is `within`).
__device__ void descend(const RowInfo& r, int mode, Prefix within, unsigned limit, double target,
                        bool strict, SampleShared& sm) {
    const int tid = threadIdx.x;
    uint32_t prefix_q = 0;
    int bits = 0;
    if (tid == 0) {
        sm.base_w = 0.0;
        sm.base_c = 0;
    }
    unsigned bucket_count = 0;
    for (int level = 0; level < 3; ++level) {
        const int shift = 16 - 8 * level;
        if (tid < 256) {
            sm.hist_w[tid] = 0.0;
            sm.hist_c[tid] = 0;
        }
        __syncthreads();
        for (int i = tid; i < r.V; i += SM_THREADS) {
            const float l = r.row[i];
            const uint32_t k = order_key(l);
            if (!in_prefix(k, i, within)) continue;
            const uint32_t q = quant24(r, l);
            if (level > 0 && (q >> (shift + 8)) != prefix_q) continue;
            const int b = (q >> shift) & 255;
            atomicAdd(&sm.hist_c[b], 1u);
            if (mode != 2) unsafeAtomicAdd(&sm.hist_w[b], weight_of(r, l, mode));
        }
        __syncthreads();
        if (tid == 0) {
            double cw = sm.base_w;
            unsigned cc = sm.base_c;
            int chosen = -1, lowest = -1;
            for (int b = 255; b >= 0; --b) {
                if (sm.hist_c[b] == 0) continue;
                lowest = b;
                const double nw = cw + sm.hist_w[b];
                const unsigned nc = cc + sm.hist_c[b];
                const bool cross = mode != 2 && (strict ? nw > target : nw >= target);
                if (cross || nc >= limit) {
                    chosen = b;
                    break;
                }
                cw = nw;
                cc = nc;
            }
            if (chosen < 0 && level > 0) {
                // the parent bucket crossed but, summed in this order, its parts do not: the
                // crossing element is the last one
                chosen = lowest;
                cw -= sm.hist_w[lowest];
                cc -= sm.hist_c[lowest];
            }
            sm.chosen = chosen;
            if (chosen >= 0) {
                sm.base_w = cw;
                sm.base_c = cc;
            } else {
                sm.res = within;
                sm.res_count = cc;
                sm.found = 0;
            }
        }
        __syncthreads();
        if (sm.chosen < 0) return;
        prefix_q = (prefix_q << 8) | (uint32_t)sm.chosen;
        bits = 8 * (level + 1);
        bucket_count = sm.hist_c[sm.chosen];
        __syncthreads();
        if (bucket_count <= SM_LIST) break;
    }
    const int qshift = 24 - bits;
    if (bucket_count <= SM_LIST) {
        if (tid == 0) sm.n_list = 0;
        __syncthreads();
        for (int i = tid; i < r.V; i += SM_THREADS) {
            const float l = r.row[i];
            const uint32_t k = order_key(l);
            if (!in_prefix(k, i, within)) continue;
            if ((quant24(r, l) >> qshift) != prefix_q) continue;
            const unsigned pos = atomicAdd(&sm.n_list, 1u);
            if (pos < SM_LIST) {
                sm.list_idx[pos] = i;
                sm.list_key[pos] = k;
            }
        }
        __syncthreads();
        const unsigned n = min(sm.n_list, (unsigned)SM_LIST);
        if ((unsigned)tid < n) {
            const uint32_t k = sm.list_key[tid];
            const int idx = sm.list_idx[tid];
            unsigned rank = 0;
            for (unsigned j = 0; j < n; ++j) {
                const uint32_t kj = sm.list_key[j];
                rank += (kj > k || (kj == k && sm.list_idx[j] < idx)) ? 1u : 0u;
            }
            sm.sorted_idx[rank] = idx;
            sm.sorted_key[rank] = k;
            sm.sorted_w[rank] = weight_of(r, key_value(k), mode);
        }
        __syncthreads();
        if (tid == 0) {
            double cw = sm.base_w;
            unsigned cc = sm.base_c;
            unsigned hit = n - 1;
            for (unsigned j = 0; j < n; ++j) {
                cw += sm.sorted_w[j];
                cc += 1;
                const bool cross = mode != 2 && (strict ? cw > target : cw >= target);
                if (cross || cc >= limit) {
                    hit = j;
                    break;
                }
            }
            sm.res = Prefix{sm.sorted_key[hit], sm.sorted_idx[hit]};
            sm.res_count = sm.base_c + hit + 1;
            sm.found = 1;
        }
        __syncthreads();
        return;
    }
    // More than SM_LIST elements share 24 quantised bits (many equal or nearly equal logits):
    // walk the distinct values of the bucket in descending order, a group of equals at a time.
    uint64_t below = 0x100000000ull;
    uint32_t last_key = 0;
    bool any = false;
    for (;;) {
        unsigned kmax = 0;
        bool have = false;
        for (int i = tid; i < r.V; i += SM_THREADS) {
            const float l = r.row[i];
            const uint32_t k = order_key(l);
            if ((uint64_t)k >= below || !in_prefix(k, i, within)) continue;
            if ((quant24(r, l) >> qshift) != prefix_q) continue;
            if (!have || k > kmax) kmax = k;
            have = true;
        }
        const unsigned cnt_have = block_sum_u32(have ? 1u : 0u, sm);
        if (cnt_have == 0) break;
        kmax = block_max_u32(have ? kmax : 0u, sm);
        unsigned ties = 0;
        for (int i = tid; i < r.V; i += SM_THREADS)
            ties += (order_key(r.row[i]) == kmax && in_prefix(kmax, i, within)) ? 1u : 0u;
        ties = block_sum_u32(ties, sm);
        const double w = weight_of(r, key_value(kmax), mode);
        const double bw = sm.base_w;
        const unsigned bc = sm.base_c;
        // smallest t in [1, ties] at which the walk stops, or 0
        unsigned t = 0;
        if (limit > bc && limit - bc <= ties) t = limit - bc;
        if (mode != 2 && w > 0.0) {
            double guess = floor((target - bw) / w);
            if (guess < 0.0) guess = 0.0;
            if (guess < (double)ties + 2.0) {
                unsigned tw = (unsigned)guess;
                tw = tw > 2 ? tw - 2 : 1;
                for (; tw <= ties; ++tw) {
                    const double s = bw + (double)tw * w;
                    if (strict ? s > target : s >= target) break;
                }
                if (tw <= ties && (t == 0 || tw < t)) t = tw;
            }
        }
        any = true;
        last_key = kmax;
        if (t > 0) {
            const int idx = nth_tie(r, kmax, within, t, sm);
            if (tid == 0) {
                sm.res = Prefix{kmax, idx};
                sm.res_count = bc + t;
                sm.found = 1;
            }
            __syncthreads();
            return;
        }
        __syncthreads();
        if (tid == 0) {
            sm.base_w = bw + (double)ties * w;
            sm.base_c = bc + ties;
        }
        __syncthreads();
        below = kmax;
    }
    if (tid == 0) {
        sm.res = any ? Prefix{last_key, 0x7fffffff} : within;
        sm.res_count = sm.base_c;
        sm.found = any ? 1 : 0;
    }
    __syncthreads();
}

__device__ __forceinline__ uint64_t xorshift64(uint64_t x) {   // picolm/sampler.c:10-17
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return x;
}

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(const float* __restrict__ logits, int64_t ld,
                                                           int V, float temperature, int top_k,
                                                           float top_p, float min_p,
                                                           uint64_t* __restrict__ rng_states,
                                                           const int32_t* __restrict__ state_index,
                                                           int32_t* __restrict__ out) {
    __shared__ SampleShared sm;
    __shared__ float sf[SM_WAVES];
    __shared__ int si[SM_WAVES];
    const int tid = threadIdx.x;
    RowInfo r;
    r.row = logits + (int64_t)blockIdx.x * ld;
    r.V = V;
    // maximum (first index) and minimum
    float best = -INFINITY, lo = INFINITY;
    int best_i = 0x7fffffff;
    for (int i = tid; i < V; i += SM_THREADS) {
        const float v = r.row[i];
        if (v > best || best_i == 0x7fffffff) {
            best = v;
            best_i = i;
        }
        lo = fminf(lo, v);
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(best_i, o, WAVE);
        if (oi != 0x7fffffff && (best_i == 0x7fffffff || ov > best || (ov == best && oi < best_i))) {
            best = ov;
            best_i = oi;
        }
        lo = fminf(lo, __shfl_xor(lo, o, WAVE));
    }
    if (tid % WAVE == 0) {
        sf[tid / WAVE] = best;
        si[tid / WAVE] = best_i;
    }
    __syncthreads();
    for (int w = 0; w < SM_WAVES; ++w) {
        if (si[w] != 0x7fffffff && (best_i == 0x7fffffff || sf[w] > best || (sf[w] == best && si[w] < best_i))) {
            best = sf[w];
            best_i = si[w];
        }
    }
    __syncthreads();
    if (tid % WAVE == 0) sf[tid / WAVE] = lo;
    __syncthreads();
    for (int w = 0; w < SM_WAVES; ++w) lo = fminf(lo, sf[w]);
    const int top_token = best_i == 0x7fffffff ? 0 : best_i;
    if (!(temperature > 0.0f)) {                                   // sampler.c:50
        if (tid == 0) out[blockIdx.x] = top_token;
        return;
    }
    r.lmin = lo;
    r.lmax = (double)best;
    r.qscale = best > lo ? 16777216.0 / ((double)best - (double)lo) : 0.0;
    r.inv_t = 1.0 / (double)temperature;

    Prefix kept = PREFIX_ALL;
    unsigned kept_n = (unsigned)V;
    const unsigned k_limit = (top_k > 0 && top_k < V) ? (unsigned)top_k : (unsigned)V;   // sampler.c:70-73
    const bool use_p = top_p < 1.0f;
    if (use_p || k_limit < (unsigned)V) {                          // sampler.c:76-82
        double Z = 0.0;
        if (use_p) {
            double z = 0.0;
            for (int i = tid; i < V; i += SM_THREADS) z += weight_of(r, r.row[i], 0);
            Z = block_sum_f64(z, sm);
        }
        descend(r, use_p ? 0 : 2, PREFIX_ALL, k_limit, (double)top_p * Z, false, sm);
        kept = sm.res;
        kept_n = sm.res_count;
        __syncthreads();
    }
    if (min_p > 0.0f && kept_n > 1) {                              // sampler.c:85-95
        unsigned kmin = 0xffffffffu;
        for (int i = tid; i < V; i += SM_THREADS) {
            const float l = r.row[i];
            const uint32_t k = order_key(l);
            if (in_prefix(k, i, kept) && weight_of(r, l, 0) >= (double)min_p) kmin = min(kmin, k);
        }
        const unsigned any = block_sum_u32(kmin != 0xffffffffu ? 1u : 0u, sm);
        kmin = block_min_u32(kmin, sm);
        if (any == 0)
            kept = Prefix{order_key(best), top_token};             // keep at least the top token
        else if (kmin > kept.key)
            kept = Prefix{kmin, 0x7fffffff};
    }
    // sampler.c:98-121: weights p^(1/T) over the kept ones, a uniform r, the first running sum > r
    double wsum = 0.0;
    for (int i = tid; i < V; i += SM_THREADS) {
        const float l = r.row[i];
        if (in_prefix(order_key(l), i, kept)) wsum += weight_of(r, l, 1);
    }
    const double W = block_sum_f64(wsum, sm);
    const int sidx = state_index ? state_index[blockIdx.x] : blockIdx.x;
    const uint64_t x = xorshift64(rng_states[sidx]);
    const float rnd = (float)(x >> 11) / 9007199254740992.0f;      // sampler.c:19-21
    descend(r, 1, kept, 0xffffffffu, (double)rnd * W, true, sm);
    if (tid == 0) {
        out[blockIdx.x] = (sm.found && sm.res.idx != 0x7fffffff) ? sm.res.idx : top_token;
        rng_states[sidx] = x;
    }
}

extern "C" int picolm_sample(const float* logits, int64_t ld, int n_rows, int V, float temperature,
                             int top_k, float top_p, float min_p, uint64_t* rng_states,
                             const int32_t* state_index, int32_t* out, hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%lld", n_rows, V,
                   (long long)ld);
    PICOLM_REQUIRE(temperature <= 0.0f || rng_states != nullptr, "sample: a temperature needs generator states");
    PICOLM_REQUIRE(top_p > 0.0f || temperature <= 0.0f, "sample: top_p must be positive, got %g", top_p);
    if (n_rows == 0) return 0;
    sample_kernel<<<dim3(n_rows), dim3(SM_THREADS), 0, stream>>>(logits, ld, V, temperature, top_k, top_p, min_p,
                                                               rng_states, state_index, out);
    PICOLM_LAUNCH_CHECK("sample");
    return 0;
}
