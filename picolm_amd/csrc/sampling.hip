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
#include <mutex>

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

// The same two kernels over scratch memory that belongs to the library: a file-scope array in
// device memory, PICOLM_ARGMAX_STATIC_FLOATS floats (256 KiB) that each GPU the library runs on
// holds until the process ends.  The array's name is a host-side handle only; its address on a
// device is asked for once per device, with that device current, and kept.
#define PICOLM_ARGMAX_STATIC_FLOATS 65536
#define PICOLM_MAX_DEVICES 64
static __device__ __align__(256) float g_argmax_scratch[PICOLM_ARGMAX_STATIC_FLOATS];
static float* g_argmax_scratch_ptr[PICOLM_MAX_DEVICES];      // per device, null until asked for
static std::mutex g_argmax_scratch_mutex;

static int argmax_static_scratch(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    PICOLM_REQUIRE(e == hipSuccess, "argmax_static: no current device: %s", hipGetErrorString(e));
    PICOLM_REQUIRE(dev >= 0 && dev < PICOLM_MAX_DEVICES, "argmax_static: device %d is beyond the %d this library keeps scratch for",
                   dev, PICOLM_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_argmax_scratch_mutex);
    if (g_argmax_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_argmax_scratch));
        PICOLM_REQUIRE(e == hipSuccess && p != nullptr, "argmax_static: no address for the scratch array on device %d: %s", dev,
                       hipGetErrorString(e));
        g_argmax_scratch_ptr[dev] = (float*)p;
    }
    *out = g_argmax_scratch_ptr[dev];
    return 0;
}

extern "C" int picolm_argmax_static_max_floats(void) { return PICOLM_ARGMAX_STATIC_FLOATS; }

extern "C" int picolm_argmax_static(const float* logits, int32_t* out, int n_rows, int V, int64_t ld,
                                    hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax_static: bad sizes rows=%d V=%d ld=%lld", n_rows, V,
                   (long long)ld);
    PICOLM_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: null logits or output");
    PICOLM_REQUIRE(n_rows <= 65535, "argmax_static: %d rows exceed the grid", n_rows);
    const int64_t need = 2 * (int64_t)n_rows * ceil_div(V, ARGMAX_SLICE);
    PICOLM_REQUIRE(need <= PICOLM_ARGMAX_STATIC_FLOATS,
                   "argmax_static: %d rows of %d logits need %lld floats of scratch, the library's array holds %d "
                   "(picolm_argmax takes a buffer of any size)", n_rows, V, (long long)need, PICOLM_ARGMAX_STATIC_FLOATS);
    if (n_rows == 0) return 0;
    float* scratch = nullptr;
    if (int rc = argmax_static_scratch(&scratch)) return rc;
    // every entry that the second kernel reads is written by the first, so what an earlier call
    // left in the array needs no clearing
    return picolm_argmax(logits, out, n_rows, V, ld, scratch, stream);
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

// Every thread of the workgroup visits its share of the row: f(index, logit).  A row that starts
// on a 16-byte boundary is read four values a load, several loads in flight.
template <typename F>
__device__ __forceinline__ void for_each_logit(const RowInfo& r, F f) {
    const int tid = threadIdx.x;
    int done = 0;
    if (((uintptr_t)r.row & 15) == 0) {
        const float4* p = (const float4*)r.row;
        const int n4 = r.V / 4;
#pragma unroll 4
        for (int j = tid; j < n4; j += SM_THREADS) {
            const float4 v = p[j];
            f(4 * j, v.x);
            f(4 * j + 1, v.y);
            f(4 * j + 2, v.z);
            f(4 * j + 3, v.w);
        }
        done = 4 * n4;
    }
    for (int i = done + tid; i < r.V; i += SM_THREADS) f(i, r.row[i]);
}

struct SampleShared {
    double hist_w[256];
    unsigned hist_c[256];
    unsigned red_u[SM_WAVES];
    int list_idx[SM_LIST];
    uint32_t list_key[SM_LIST];
    int sorted_idx[SM_LIST];
    uint32_t sorted_key[SM_LIST];
    double sorted_w[SM_LIST];
    unsigned n_list;
    int chosen;
    double base_w;
    double target;
    unsigned base_c;
    Prefix res;
    unsigned res_count;
    int found;
    unsigned bcast_u;
    int bcast_i;
};

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
// The target is `fraction` times the sum of all weights of `within`, which the first histogram
// gives (its buckets in ascending order): no pass of its own for the sum.
__device__ void descend(const RowInfo& r, int mode, Prefix within, unsigned limit, double fraction,
                        bool strict, SampleShared& sm) {
    const int tid = threadIdx.x;
    double target = 0.0;
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
        for_each_logit(r, [&](int i, float l) {
            const uint32_t k = order_key(l);
            if (!in_prefix(k, i, within)) return;
            const uint32_t q = quant24(r, l);
            if (level > 0 && (q >> (shift + 8)) != prefix_q) return;
            const int b = (q >> shift) & 255;
            atomicAdd(&sm.hist_c[b], 1u);
            if (mode != 2) unsafeAtomicAdd(&sm.hist_w[b], weight_of(r, l, mode));
        });
        __syncthreads();
        if (level == 0) {
            if (tid == 0) {
                double total = 0.0;
                for (int b = 0; b < 256; ++b) total += sm.hist_w[b];
                sm.target = fraction * total;
            }
            __syncthreads();
            target = sm.target;
        }
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
        for_each_logit(r, [&](int i, float l) {
            const uint32_t k = order_key(l);
            if (!in_prefix(k, i, within)) return;
            if ((quant24(r, l) >> qshift) != prefix_q) return;
            const unsigned pos = atomicAdd(&sm.n_list, 1u);
            if (pos < SM_LIST) {
                sm.list_idx[pos] = i;
                sm.list_key[pos] = k;
            }
        });
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
    for_each_logit(r, [&](int i, float v) {      // (a thread's indices come in ascending order)
        if (v > best || best_i == 0x7fffffff) {
            best = v;
            best_i = i;
        }
        lo = fminf(lo, v);
    });
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
        descend(r, use_p ? 0 : 2, PREFIX_ALL, k_limit, (double)top_p, false, sm);
        kept = sm.res;
        kept_n = sm.res_count;
        __syncthreads();
    }
    if (min_p > 0.0f && kept_n > 1) {                              // sampler.c:85-95
        unsigned kmin = 0xffffffffu;
        for_each_logit(r, [&](int i, float l) {
            const uint32_t k = order_key(l);
            if (in_prefix(k, i, kept) && weight_of(r, l, 0) >= (double)min_p) kmin = min(kmin, k);
        });
        const unsigned any = block_sum_u32(kmin != 0xffffffffu ? 1u : 0u, sm);
        kmin = block_min_u32(kmin, sm);
        if (any == 0)
            kept = Prefix{order_key(best), top_token};             // keep at least the top token
        else if (kmin > kept.key)
            kept = Prefix{kmin, 0x7fffffff};
    }
    // sampler.c:98-121: weights p^(1/T) over the kept ones, a uniform r, the first running sum > r
    const int sidx = state_index ? state_index[blockIdx.x] : blockIdx.x;
    const uint64_t x = xorshift64(rng_states[sidx]);
    const float rnd = (float)(x >> 11) / 9007199254740992.0f;      // sampler.c:19-21
    descend(r, 1, kept, 0xffffffffu, (double)rnd, true, sm);
    if (tid == 0) {
        out[blockIdx.x] = (sm.found && sm.res.idx != 0x7fffffff) ? sm.res.idx : top_token;
        rng_states[sidx] = x;
    }
}

// ---------------------------------------------------------------------------------------------
// With a top_k of a few dozen (picolm's default is 40) everything after the first cut works on
// those k elements and on the softmax denominator.  Then a row is cut into slices, one workgroup
// each: a slice leaves its maximum, its sum of exp(l - maximum) and its own k first elements in
// the descending order (the row's k first are among them); one workgroup per row then orders the
// candidates exactly and runs picolm's pipeline (sampler.c:58-121) on the first k.
#define SLICE_VALUES 4096
#define SLICE_THREADS 256
#define SLICE_PER_THREAD (SLICE_VALUES / SLICE_THREADS)
#define PICK_THREADS 1024
#define PICK_MAX_CANDIDATES 4096
#define PICK_MAX_TOP 1024

struct SliceOut {          // per row and slice
    float* max;            // [rows][slices]
    double* sum;           // [rows][slices]
    int32_t* count;        // [rows][slices]  candidates the slice left (min(k, its size))
    uint32_t* key;         // [rows][slices][k]
    int32_t* idx;          // [rows][slices][k]
};
__host__ __device__ inline size_t slice_out_bytes(int n_rows, int n_slices, int k) {
    const size_t per = (size_t)n_rows * n_slices;
    return per * 8 + per * 8 + per * 8 + per * k * 4 + per * k * 4;      // every part a multiple of 8 bytes
}
__host__ __device__ inline SliceOut slice_out_at(void* scratch, int n_rows, int n_slices, int k) {
    const size_t per = (size_t)n_rows * n_slices;
    char* p = (char*)scratch;
    SliceOut o;
    o.sum = (double*)p;
    o.max = (float*)(p + per * 8);
    o.count = (int32_t*)(p + per * 16);
    o.key = (uint32_t*)(p + per * 24);
    o.idx = (int32_t*)(p + per * 24 + per * k * 4);
    return o;
}

// One wave finds, in a histogram of 256 bins, the bin that holds the `remaining`-th element
// counted from the highest bin down, and how many elements lie in the bins above it.  The bins
// hold at least `remaining` elements.
__device__ __forceinline__ void find_bin(const unsigned* hist, unsigned remaining, int lane, unsigned& sel_bin,
                                         unsigned& sel_above, unsigned& sel_count) {
    // lane L holds bins 4L .. 4L+3; `above` counts the elements of all higher bins
    const unsigned b0 = hist[4 * lane], b1 = hist[4 * lane + 1], b2 = hist[4 * lane + 2], b3 = hist[4 * lane + 3];
    const unsigned mine = b0 + b1 + b2 + b3;
    unsigned incl = mine;          // sum over lanes >= this one
#pragma unroll
    for (int s = 1; s < WAVE; s <<= 1) {
        const unsigned other = __shfl_down(incl, s, WAVE);
        if (lane + s < WAVE) incl += other;
    }
    unsigned above = incl - mine;
    if (above < remaining && remaining <= incl) {        // one lane: the crossing is in its bins
        int bin = 4 * lane + 3;
        if (above + b3 < remaining) {
            above += b3;
            bin = 4 * lane + 2;
            if (above + b2 < remaining) {
                above += b2;
                bin = 4 * lane + 1;
                if (above + b1 < remaining) {
                    above += b1;
                    bin = 4 * lane;
                }
            }
        }
        sel_bin = (unsigned)bin;
        sel_above = above;
        sel_count = hist[bin];
    }
}

__global__ __launch_bounds__(SLICE_THREADS) void sample_slice_kernel(const float* __restrict__ logits, int64_t ld,
                                                                     int V, int k, SliceOut o) {
    __shared__ unsigned hist[256];
    __shared__ float red_f[SLICE_THREADS / WAVE];
    __shared__ double red_d[SLICE_THREADS / WAVE];
    __shared__ unsigned red_u[SLICE_THREADS / WAVE];
    __shared__ unsigned sel_bin, sel_above, sel_count, n_out;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int n_slices = gridDim.x;
    const size_t slot = (size_t)blockIdx.y * n_slices + blockIdx.x;
    const float* row = logits + (int64_t)blockIdx.y * ld;
    const int lo = blockIdx.x * SLICE_VALUES;
    const int n = min(SLICE_VALUES, V - lo);
    // a thread holds 16 adjacent values, so that threads in order hold indices in order
    float v[SLICE_PER_THREAD];
    uint32_t key[SLICE_PER_THREAD];
    const int first = tid * SLICE_PER_THREAD;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < SLICE_PER_THREAD; ++j) {
        const bool ok = first + j < n;
        v[j] = ok ? row[lo + first + j] : -INFINITY;
        key[j] = order_key(v[j]);
        if (ok) mx = fmaxf(mx, v[j]);
    }
#pragma unroll
    for (int s = WAVE / 2; s > 0; s >>= 1) mx = fmaxf(mx, __shfl_xor(mx, s, WAVE));
    if (lane == 0) red_f[wave] = mx;
    __syncthreads();
    mx = red_f[0];
#pragma unroll
    for (int w = 1; w < SLICE_THREADS / WAVE; ++w) mx = fmaxf(mx, red_f[w]);
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < SLICE_PER_THREAD; ++j)
        if (first + j < n) sum += exp((double)v[j] - (double)mx);
#pragma unroll
    for (int s = WAVE / 2; s > 0; s >>= 1) sum += __shfl_xor(sum, s, WAVE);
    if (lane == 0) red_d[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        double t = 0.0;
        for (int w = 0; w < SLICE_THREADS / WAVE; ++w) t += red_d[w];
        o.sum[slot] = t;
        o.max[slot] = mx;
        o.count[slot] = min(k, n);
        n_out = 0;
    }
    uint32_t* out_key = o.key + slot * k;
    int32_t* out_idx = o.idx + slot * k;
    if (n <= k) {                         // every element is a candidate
#pragma unroll
        for (int j = 0; j < SLICE_PER_THREAD; ++j)
            if (first + j < n) {
                out_key[first + j] = key[j];
                out_idx[first + j] = lo + first + j;
            }
        return;
    }
    // the key of the k-th element in descending order, eight bits at a time from the top
    uint32_t prefix = 0;
    unsigned remaining = (unsigned)k;      // how many of the elements that share `prefix` are taken
    int low_bits = 0;                      // bits of the key below `prefix` when the search ends
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        hist[tid] = 0;                     // (256 threads, 256 bins)
        __syncthreads();
#pragma unroll
        for (int j = 0; j < SLICE_PER_THREAD; ++j)
            if (first + j < n && (pass == 0 || (key[j] >> (shift + 8)) == prefix)) atomicAdd(&hist[(key[j] >> shift) & 255], 1u);
        __syncthreads();
        if (wave == 0) find_bin(hist, remaining, lane, sel_bin, sel_above, sel_count);
        __syncthreads();
        prefix = (prefix << 8) | sel_bin;
        remaining -= sel_above;
        const bool whole_bin = sel_count == remaining;      // all that share the prefix are taken
        __syncthreads();
        if (whole_bin) {
            low_bits = shift;
            break;
        }
    }
    // everything above the k-th key, and of its equals the first `remaining` by index (if the
    // search ended early, `kth` is the least key with the prefix and all its "equals" are taken)
    const uint32_t kth = prefix;
    unsigned equals = 0;
#pragma unroll
    for (int j = 0; j < SLICE_PER_THREAD; ++j) {
        key[j] >>= low_bits;
        equals += (first + j < n && key[j] == kth) ? 1u : 0u;
    }
    unsigned scan = equals;                // inclusive over the lanes of the wave
#pragma unroll
    for (int s = 1; s < WAVE; s <<= 1) {
        const unsigned other = __shfl_up(scan, s, WAVE);
        if (lane >= s) scan += other;
    }
    if (lane == WAVE - 1) red_u[wave] = scan;
    __syncthreads();
    unsigned before = scan - equals;       // equals in threads before this one
    for (int w = 0; w < wave; ++w) before += red_u[w];
#pragma unroll
    for (int j = 0; j < SLICE_PER_THREAD; ++j) {
        if (first + j >= n) continue;
        bool take = key[j] > kth;
        if (key[j] == kth) take = before++ < remaining;
        if (take) {
            const unsigned pos = atomicAdd(&n_out, 1u);      // exactly k of them
            out_key[pos] = order_key(v[j]);
            out_idx[pos] = lo + first + j;
        }
    }
}

// A candidate as one number whose descending order is the pipeline's: the logit's key above,
// the token id below, inverted so that of equal logits the lower id comes first.  0: no candidate.
__device__ __forceinline__ uint64_t candidate(uint32_t key, int idx) {
    return ((uint64_t)key << 32) | (uint32_t)(0x7fffffff - idx);
}
__device__ __forceinline__ uint32_t candidate_key(uint64_t c) { return (uint32_t)(c >> 32); }
__device__ __forceinline__ int candidate_idx(uint64_t c) { return 0x7fffffff - (int)(uint32_t)c; }

struct PickShared {
    uint64_t cand[PICK_MAX_CANDIDATES];
    uint64_t unordered[PICK_MAX_TOP];
    uint64_t top[PICK_MAX_TOP];
    double z_part[PICK_THREADS];       // a slice's share of the softmax denominator
};

__global__ __launch_bounds__(PICK_THREADS) void sample_pick_kernel(SliceOut o, int n_slices, int k, float temperature,
                                                                   float top_p, float min_p,
                                                                   uint64_t* __restrict__ rng_states,
                                                                   const int32_t* __restrict__ state_index,
                                                                   int32_t* __restrict__ out) {
    __shared__ PickShared sm;
    __shared__ unsigned hist[256];
    __shared__ unsigned sel_bin, sel_above, sel_count;
    __shared__ int n_valid, n_gathered;
    const int tid = threadIdx.x;
    const size_t slot0 = (size_t)blockIdx.x * n_slices;
    const int n_slots = n_slices * k;
    const int n_padded = (n_slots + 3) & ~3;
    // asked for early: the generator's state, and the slices' maxima and sums
    const int sidx = state_index ? state_index[blockIdx.x] : blockIdx.x;
    const uint64_t state = tid == 0 ? rng_states[sidx] : 0;
    float s_max = -INFINITY;
    double s_sum = 0.0;
    if (tid < n_slices) {                                  // (n_slices * k <= 4096 and k >= 1)
        s_max = o.max[slot0 + tid];
        s_sum = o.sum[slot0 + tid];
    }
    if (tid == 0) n_valid = n_gathered = 0;
    __syncthreads();
    int mine = 0;
    for (int c = tid; c < n_padded; c += PICK_THREADS) {
        const int s = c / k, j = c % k;
        const bool ok = c < n_slots && j < o.count[slot0 + s];
        sm.cand[c] = ok ? candidate(o.key[(slot0 + s) * k + j], o.idx[(slot0 + s) * k + j]) : 0ull;
        mine += ok ? 1 : 0;
    }
    if (mine) atomicAdd(&n_valid, mine);
    __syncthreads();
    const int n_top = min(k, n_valid);
    // the k-th candidate in descending order, eight bits at a time from the top
    uint64_t kth = 1;                          // (every candidate is at least 1)
    if (n_valid > k) {
        uint64_t prefix = 0;
        unsigned remaining = (unsigned)k;
        for (int pass = 0; pass < 8; ++pass) {
            const int shift = 56 - 8 * pass;
            if (tid < 256) hist[tid] = 0;
            __syncthreads();
            for (int c = tid; c < n_slots; c += PICK_THREADS) {
                const uint64_t me = sm.cand[c];
                if (me != 0ull && (pass == 0 || (me >> (shift + 8)) == prefix)) atomicAdd(&hist[(unsigned)(me >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid < WAVE) find_bin(hist, remaining, tid, sel_bin, sel_above, sel_count);
            __syncthreads();
            prefix = (prefix << 8) | sel_bin;
            remaining -= sel_above;
            const bool whole_bin = sel_count == remaining;      // all that share the prefix are taken
            __syncthreads();
            if (whole_bin) {
                prefix <<= shift;
                break;
            }
        }
        kth = prefix;
    }
    // the first k, gathered in any order, then put in order: a candidate's place is the number
    // of greater ones among them
    for (int c = tid; c < n_slots; c += PICK_THREADS) {
        const uint64_t me = sm.cand[c];
        if (me != 0ull && me >= kth) sm.unordered[atomicAdd(&n_gathered, 1)] = me;
    }
    __syncthreads();
    for (int c = tid; c < n_top; c += PICK_THREADS) {
        const uint64_t me = sm.unordered[c];
        int rank = 0;
        for (int j = 0; j < n_top; ++j) rank += sm.unordered[j] > me ? 1 : 0;
        sm.top[rank] = me;
    }
    __syncthreads();
    // the candidates' place now holds the weights of the first k: exp(l - max), exp((l - max) / T)
    double* w_plain = (double*)sm.cand;
    double* w_temp = w_plain + PICK_MAX_TOP;
    // the row's maximum is the first candidate's logit; every thread weighs candidates and slices
    const double lmax = (double)key_value(candidate_key(sm.top[0]));
    const double inv_t = 1.0 / (double)temperature;
    for (int j = tid; j < n_top; j += PICK_THREADS) {
        const double x = (double)key_value(candidate_key(sm.top[j])) - lmax;
        w_plain[j] = exp(x);
        w_temp[j] = exp(x * inv_t);
    }
    if (tid < n_slices) sm.z_part[tid] = s_sum * exp((double)s_max - lmax);
    __syncthreads();
    if (tid != 0) return;
    double Z = 0.0;                                                // the softmax denominator
    for (int s = 0; s < n_slices; ++s) Z += sm.z_part[s];
    const int top_token = candidate_idx(sm.top[0]);
    int kept = n_top;                                              // sampler.c:70-73
    if (top_p < 1.0f) {                                            // sampler.c:76-82
        const double target = (double)top_p * Z;
        double cum = 0.0;
        bool hit = false;
        for (int j0 = 0; j0 < n_top && !hit; j0 += 8) {            // eight weights are read at a time
            double w[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) w[e] = w_plain[min(j0 + e, n_top - 1)];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                cum += w[e];
                if (!hit && j0 + e < n_top && cum >= target) {
                    kept = j0 + e + 1;
                    hit = true;
                }
            }
        }
    }
    if (min_p > 0.0f && kept > 1) {                                // sampler.c:85-95
        int m = 0;
        while (m < kept && w_plain[m] >= (double)min_p) ++m;
        kept = m > 0 ? m : 1;                                      // keep at least the top token
    }
    // sampler.c:98-121
    double W = 0.0;
    for (int j0 = 0; j0 < kept; j0 += 8) {
        double w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = w_temp[min(j0 + e, kept - 1)];
#pragma unroll
        for (int e = 0; e < 8; ++e) W += j0 + e < kept ? w[e] : 0.0;
    }
    const uint64_t x = xorshift64(state);
    const float rnd = (float)(x >> 11) / 9007199254740992.0f;      // sampler.c:19-21
    const double target = (double)rnd * W;
    int chosen = top_token;
    double cum = 0.0;
    bool hit = false;
    for (int j0 = 0; j0 < kept && !hit; j0 += 8) {
        double w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = w_temp[min(j0 + e, kept - 1)];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            cum += w[e];
            if (!hit && j0 + e < kept && cum > target) {
                chosen = candidate_idx(sm.top[j0 + e]);
                hit = true;
            }
        }
    }
    out[blockIdx.x] = chosen;
    rng_states[sidx] = x;
}

// Whether the sliced kernels take this case, and the scratch memory they need then (0: they do not).
extern "C" int picolm_sample_scratch_bytes(int n_rows, int V, float temperature, int top_k) {
    if (!(temperature > 0.0f) || top_k <= 0 || top_k >= V || top_k > PICK_MAX_TOP || n_rows <= 0) return 0;
    const int n_slices = ceil_div(V, SLICE_VALUES);
    if ((int64_t)n_slices * top_k > PICK_MAX_CANDIDATES || n_slices > PICK_THREADS) return 0;
    const size_t bytes = slice_out_bytes(n_rows, n_slices, top_k);
    return bytes < (1u << 30) ? (int)bytes : 0;
}

// `scratch`: picolm_sample_scratch_bytes(...) bytes of device memory, 8-byte aligned, or null;
// without it, or where that function says 0, one workgroup per row does all the work.
extern "C" int picolm_sample(const float* logits, int64_t ld, int n_rows, int V, float temperature,
                             int top_k, float top_p, float min_p, uint64_t* rng_states,
                             const int32_t* state_index, int32_t* out, void* scratch, int64_t scratch_bytes,
                             hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%lld", n_rows, V,
                   (long long)ld);
    PICOLM_REQUIRE(temperature <= 0.0f || rng_states != nullptr, "sample: a temperature needs generator states");
    PICOLM_REQUIRE(top_p > 0.0f || temperature <= 0.0f, "sample: top_p must be positive, got %g", top_p);
    if (n_rows == 0) return 0;
    const int need = picolm_sample_scratch_bytes(n_rows, V, temperature, top_k);
    if (need > 0 && scratch != nullptr && n_rows <= 65535) {
        PICOLM_REQUIRE(scratch_bytes >= need && ((uintptr_t)scratch & 7) == 0,
                       "sample: the scratch buffer holds %lld bytes, %lld are needed (8-byte aligned)",
                       (long long)scratch_bytes, (long long)need);
        const int n_slices = ceil_div(V, SLICE_VALUES);
        const SliceOut o = slice_out_at(scratch, n_rows, n_slices, top_k);
        sample_slice_kernel<<<dim3(n_slices, n_rows), dim3(SLICE_THREADS), 0, stream>>>(logits, ld, V, top_k, o);
        PICOLM_LAUNCH_CHECK("sample");
        sample_pick_kernel<<<dim3(n_rows), dim3(PICK_THREADS), 0, stream>>>(o, n_slices, top_k, temperature, top_p,
                                                                           min_p, rng_states, state_index, out);
        PICOLM_LAUNCH_CHECK("sample");
        return 0;
    }
    sample_kernel<<<dim3(n_rows), dim3(SM_THREADS), 0, stream>>>(logits, ld, V, temperature, top_k, top_p, min_p,
                                                               rng_states, state_index, out);
    PICOLM_LAUNCH_CHECK("sample");
    return 0;
}
