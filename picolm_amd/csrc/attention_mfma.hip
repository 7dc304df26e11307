// bf16 attention over the paged cache on the matrix cores of gfx950, head sizes in multiples of 32
// up to 256.
//
// Both kernels compute S^T = K Q^T with 32x32x16 MFMAs, so that an accumulator lane holds one
// query (column) and 16 keys (rows): a query's maximum and sum are an in-lane reduction plus
// one exchange with lane^32, and the rescaling of the output accumulator O^T = V^T P^T is a
// per-lane scalar.  The rows of an S^T tile are a permutation of its 32 keys, chosen so that a
// lane's 16 accumulator values are 16 consecutive keys; P^T then feeds the second MFMA
// straight from registers.  The cache pages hold K and V^T in the order of the MFMA operands
// (k_page_offset, v_page_offset), so that a wave-wide load of an operand reads 1 KB in a row.
// Softmax statistics are float, in the base-2 domain: p = exp2(s*scale*log2e - m).
//
//   prefill: a workgroup of 4 waves shares K and V^T tiles of one page through LDS, where they
//            arrive straight from the cache (global_load_lds_dwordx4); a wave owns 32 new tokens
//            of one query head and takes a page as two tiles of 32 keys, one tile's softmax
//            written between the other tile's products; with grouped heads the waves of a
//            workgroup take different heads of the group, so a page is loaded once per group.
//   decode : a wave streams its own pages straight from global memory into MFMA operands
//            (columns = the query heads of one KV group); the 4 waves of a workgroup take
//            pages in turn and merge through LDS; the chunks of a sequence leave partial
//            results in a buffer, and the workgroup that finishes last adds them up itself.
#include <utility>
#include "common.h"
#include "api.h"
#include "attention.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f
#define LAZY_MAX_STEP 8.0f

__device__ __forceinline__ bf16x8 ldg8(const bf16_t* p) { return *(const bf16x8*)p; }
// N chunks of a tile of keys or values, 512 elements apart (a wave's load is one contiguous KB).
// `once`: no other workgroup of the launch reads them, so they are marked non-temporal and pass the
// caches without displacing anything (a sweep over memory is a seventh faster that way).
template <int N>
__device__ __forceinline__ void load_tile_chunks(bf16x8 (&dst)[N], const bf16_t* p, bool once) {
    if (once) {
#pragma unroll
        for (int s = 0; s < N; ++s) dst[s] = __builtin_nontemporal_load((const bf16x8*)(p + 512 * s));
    } else {
#pragma unroll
        for (int s = 0; s < N; ++s) dst[s] = ldg8(p + 512 * s);
    }
}
__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
    return z;
}
// key (within the tile) of accumulator element e of a lane in half h
__device__ __forceinline__ int key_of_elem(int e, int h) { return 16 * (e >> 3) + 8 * h + (e & 7); }

__device__ __forceinline__ __bf16 to_bf16(float f) { return (__bf16)f; }      // the hardware's round-to-nearest-even

// 2^x as the hardware's one instruction.  exp2f() wraps it in a range check and two scalings so
// that results below 2^-126 come out as denormals; a probability that small adds nothing to a sum
// of float probabilities whose largest is near 1, and zero is as good.
__device__ __forceinline__ float exp2_flushing(float x) { return __builtin_amdgcn_exp2f(x); }


// A value's maximum or sum over a lane and the lane 32 further on (or back): one swap of the
// wave's halves (both results of it hold the lower half's value and the upper half's), no LDS.
__device__ __forceinline__ float max_of_halves(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_of_halves(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The softmax of one S^T tile (32 keys) of a wave in pieces, so that the pieces can be written
// between the matrix products of another tile: mask and maximum of some elements; then the
// reference point of the exponentials; then the probabilities of some elements, as operands of
// the second product; then the sum.
struct TileSoftmax {
    float mx, m_new, alpha, sum;
    bool rescale;
};
template <bool MASKED>
__device__ __forceinline__ void softmax_mask_max(f32x16& S, int e0, int n, int key0, int qpos, bool q_ok, int window, int h, TileSoftmax& t) {
#pragma unroll
    for (int e = e0; e < e0 + n; ++e) {
        if (MASKED) {
            const int key = key0 + key_of_elem(e, h);
            const bool vis = q_ok && key <= qpos && (window <= 0 || qpos - key < window);
            S[e] = vis ? S[e] : NEG_BIG;
        }                               // else every key of the page is visible to every query of the wave
        t.mx = fmaxf(t.mx, S[e]);
    }
}
// m_run is the reference point of the exponentials, not necessarily the maximum: it follows the
// maximum only when that has grown by more than LAZY_MAX_STEP (in powers of two), so that most
// tiles leave it alone and O^T need not be rescaled.  The result is the same in exact arithmetic;
// probabilities may reach 2^LAZY_MAX_STEP instead of 1 meanwhile.  The scores stay unscaled (the
// scale is positive, so their order is that of the scaled ones): the scale goes into the
// exponent's multiply-add.
__device__ __forceinline__ void softmax_reference(TileSoftmax& t, float m_run, float scale2) {
    const float mx = max_of_halves(t.mx) * scale2;
    const bool grow = mx > m_run + LAZY_MAX_STEP;
    t.m_new = grow ? mx : m_run;
    t.alpha = grow ? exp2_flushing(m_run - t.m_new) : 1.0f;
    t.rescale = __any(grow);
    t.sum = 0.f;
}
template <bool MASKED>
__device__ __forceinline__ void softmax_exp(const f32x16& S, int e0, int n, float scale2, TileSoftmax& t, bf16x8 (&Pf)[2]) {
#pragma unroll
    for (int e = e0; e < e0 + n; ++e) {
        const float p = (!MASKED || S[e] > 0.5f * NEG_BIG) ? exp2_flushing(fmaf(S[e], scale2, -t.m_new)) : 0.f;
        t.sum += p;
        Pf[e / 8][e % 8] = to_bf16(p);
    }
}
__device__ __forceinline__ void softmax_finish(TileSoftmax& t, float& m_run, float& l_run) {
    l_run = l_run * t.alpha + sum_of_halves(t.sum);
    m_run = t.m_new;
}

// v *= alpha, every element in the register it is in.  (Written as plain C++ the compiler gives
// the product registers of its own and copies all of O^T, on the path that does not rescale too.)
__device__ __forceinline__ void scale_in_place(f32x16& v, float alpha) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        float x = v[e];
        asm volatile("v_mul_f32 %0, %1, %0" : "+v"(x) : "v"(alpha));
        v[e] = x;
    }
}

// One page of one wave: scores, online softmax, and the update of O^T, a tile of 32 keys at a
// time, with one tile's softmax (vector ALU) written between the other tile's products (matrix
// cores) and held there, so that a wave keeps both busy: S1 = K1 Q^T beside softmax(S0), then
// O^T += V0^T P0^T beside softmax(S1).  KOP(t, s) returns the K operand of tile t, k-step s;
// VOP(dt, t, ks) the V^T operand of column block dt.
template <int D, bool MASKED, typename KOP, typename VOP>
__device__ __forceinline__ void attend_page(const bf16x8 (&Qf)[D / 16], f32x16 (&O)[D / 32], float& m_run,
                                            float& l_run, int key0, int qpos, bool q_ok, int window,
                                            float scale2, int h, KOP kop, VOP vop) {
    constexpr int NP = D / 16;                  // products of a tile, in either role
    static_assert(NP % 2 == 0, "half of the products see the maximum, half the exponentials");
    constexpr int NH = NP / 2;                  // the 16 elements of a lane go between them in NH pieces each time:
    // piece s covers elements 16 s / NH .. 16 (s + 1) / NH (as even as NH allows)
    f32x16 S0, S1;
#pragma unroll
    for (int e = 0; e < 16; ++e) S0[e] = 0.f, S1[e] = 0.f;
    // (every operand is asked for two products early and held there: the compiler, left alone,
    // asks for all of a tile's operands at once and runs out of registers)
    bf16x8 ahead = kop(0, 0), ahead2 = kop(0, 1);
#pragma unroll
    for (int s = 0; s < NP; ++s) {
        const bf16x8 now = ahead;
        ahead = ahead2;
        ahead2 = s + 2 < NP ? kop(0, s + 2) : kop(1, s + 2 - NP);
        S0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(now, Qf[s], S0, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
    TileSoftmax t;
    bf16x8 P0[2], P1[2];
    t.mx = NEG_BIG;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NP; ++s) {
        const bf16x8 now = ahead;
        ahead = ahead2;
        ahead2 = s + 2 < NP ? kop(1, s + 2) : vop((s + 2 - NP) / 2, 0, (s + 2 - NP) % 2);
        S1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(now, Qf[s], S1, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (16 % NH == 0) {
            constexpr int PIECE = 16 / NH;
            if (s < NH) softmax_mask_max<MASKED>(S0, PIECE * s, PIECE, key0, qpos, q_ok, window, h, t);
            if (s == NH - 1) softmax_reference(t, m_run, scale2);
            if (s >= NH) softmax_exp<MASKED>(S0, PIECE * (s - NH), PIECE, scale2, t, P0);
        } else {
            if (s < NH) softmax_mask_max<MASKED>(S0, 16 * s / NH, 16 * (s + 1) / NH - 16 * s / NH, key0, qpos, q_ok, window, h, t);
            if (s == NH - 1) softmax_reference(t, m_run, scale2);
            if (s >= NH) softmax_exp<MASKED>(S0, 16 * (s - NH) / NH, 16 * (s - NH + 1) / NH - 16 * (s - NH) / NH, scale2, t, P0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    softmax_finish(t, m_run, l_run);
    if (t.rescale) {
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) scale_in_place(O[dt], t.alpha);
    }
    t.mx = NEG_BIG;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NP; ++s) {
        const bf16x8 now = ahead;
        ahead = ahead2;
        ahead2 = s + 2 < NP ? vop((s + 2) / 2, 0, (s + 2) % 2) : vop((s + 2 - NP) / 2, 1, (s + 2 - NP) % 2);
        O[s / 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(now, P0[s % 2], O[s / 2], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (16 % NH == 0) {
            constexpr int PIECE = 16 / NH;
            if (s < NH) softmax_mask_max<MASKED>(S1, PIECE * s, PIECE, key0 + 32, qpos, q_ok, window, h, t);
            if (s == NH - 1) softmax_reference(t, m_run, scale2);
            if (s >= NH) softmax_exp<MASKED>(S1, PIECE * (s - NH), PIECE, scale2, t, P1);
        } else {
            if (s < NH) softmax_mask_max<MASKED>(S1, 16 * s / NH, 16 * (s + 1) / NH - 16 * s / NH, key0 + 32, qpos, q_ok, window, h, t);
            if (s == NH - 1) softmax_reference(t, m_run, scale2);
            if (s >= NH) softmax_exp<MASKED>(S1, 16 * (s - NH) / NH, 16 * (s - NH + 1) / NH - 16 * (s - NH) / NH, scale2, t, P1);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    softmax_finish(t, m_run, l_run);
    if (t.rescale) {
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) scale_in_place(O[dt], t.alpha);
    }
#pragma unroll
    for (int s = 0; s < NP; ++s) {
        const bf16x8 now = ahead;
        ahead = ahead2;
        if (s + 2 < NP) ahead2 = vop((s + 2) / 2, 1, (s + 2) % 2);
        O[s / 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(now, P1[s % 2], O[s / 2], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The same for one tile of 32 keys whose operands are already in registers (decode).
template <int D>
__device__ __forceinline__ void attend_tile(const bf16x8 (&Qf)[D / 16], const bf16x8 (&Kf)[D / 16],
                                            const bf16x8 (&Vf)[D / 32][2], f32x16 (&O)[D / 32], float& m_run,
                                            float& l_run, int key0, int key_max, int qpos, bool q_ok, int window,
                                            float scale2, int h) {
    f32x16 S;
#pragma unroll
    for (int e = 0; e < 16; ++e) S[e] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Kf[s], Qf[s], S, 0, 0, 0);
    float mx = NEG_BIG;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int key = key0 + key_of_elem(e, h);
        const bool vis = q_ok && key <= key_max && (window <= 0 || qpos - key < window);
        S[e] = vis ? S[e] * scale2 : NEG_BIG;
        mx = fmaxf(mx, S[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = exp2_flushing(m_run - m_new);
    float sum = 0.f;
    bf16x8 Pf[2];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const float p = S[e] > 0.5f * NEG_BIG ? exp2_flushing(S[e] - m_new) : 0.f;
        sum += p;
        Pf[e / 8][e % 8] = to_bf16(p);
    }
    sum += __shfl_xor(sum, 32, WAVE);
    l_run = l_run * alpha + sum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt) {
#pragma unroll
        for (int e = 0; e < 16; ++e) O[dt][e] *= alpha;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
            O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Vf[dt][ks], Pf[ks], O[dt], 0, 0, 0);
    }
}

// A lane's share of a query row as MFMA operands, taken from the float row that the qkv product
// left and rotated by the position's table row on the way (cos_t null: only rounded).  k-step s of
// a lane in wave half h covers elements 16s + 8h .. + 8.
template <int D>
__device__ __forceinline__ void rotated_q(const AttnArgs& a, const float* row, int pos, int h, bool ok, bf16x8 (&Qf)[D / 16]) {
    const float* c = a.cos_t ? a.cos_t + (size_t)pos * (D / 2) : nullptr;
    const float* sn = a.sin_t ? a.sin_t + (size_t)pos * (D / 2) : nullptr;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) Qf[s] = zero8();
    if (!ok) return;
    if (!c) {
#pragma unroll
        for (int s = 0; s < D / 16; ++s) {
            const f32x4 x0 = *(const f32x4*)(row + 16 * s + 8 * h), x1 = *(const f32x4*)(row + 16 * s + 8 * h + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                Qf[s][e] = to_bf16(x0[e]);
                Qf[s][4 + e] = to_bf16(x1[e]);
            }
        }
    } else if (a.rope_style == 0) {
#pragma unroll
        for (int s = 0; s < D / 16; ++s) {
            const int d0 = 16 * s + 8 * h;
            const f32x4 x0 = *(const f32x4*)(row + d0), x1 = *(const f32x4*)(row + d0 + 4);
            const f32x4 cc = *(const f32x4*)(c + d0 / 2), ss = *(const f32x4*)(sn + d0 / 2);
            Qf[s][0] = to_bf16(x0[0] * cc[0] - x0[1] * ss[0]);
            Qf[s][1] = to_bf16(x0[0] * ss[0] + x0[1] * cc[0]);
            Qf[s][2] = to_bf16(x0[2] * cc[1] - x0[3] * ss[1]);
            Qf[s][3] = to_bf16(x0[2] * ss[1] + x0[3] * cc[1]);
            Qf[s][4] = to_bf16(x1[0] * cc[2] - x1[1] * ss[2]);
            Qf[s][5] = to_bf16(x1[0] * ss[2] + x1[1] * cc[2]);
            Qf[s][6] = to_bf16(x1[2] * cc[3] - x1[3] * ss[3]);
            Qf[s][7] = to_bf16(x1[2] * ss[3] + x1[3] * cc[3]);
        }
    } else {
#pragma unroll
        for (int s = 0; s < D / 32; ++s) {
            const int d0 = 16 * s + 8 * h;          // below d/2; its partner is d0 + d/2, k-step s + D/32 of this lane
#pragma unroll
            for (int half4 = 0; half4 < 2; ++half4) {
                const f32x4 lo = *(const f32x4*)(row + d0 + 4 * half4), hi = *(const f32x4*)(row + d0 + D / 2 + 4 * half4);
                const f32x4 cc = *(const f32x4*)(c + d0 + 4 * half4), ss = *(const f32x4*)(sn + d0 + 4 * half4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Qf[s][4 * half4 + e] = to_bf16(lo[e] * cc[e] - hi[e] * ss[e]);
                    Qf[s + D / 32][4 * half4 + e] = to_bf16(lo[e] * ss[e] + hi[e] * cc[e]);
                }
            }
        }
    }
}

// =============================================================================================
// LDS tiles of the prefill kernel: a page's K and V^T as they lie in the cache, that is in the
// order of the MFMA operands: the 64 lanes of a wave read 64 adjacent 16-byte chunks.
//
// HALVES = 2: eight waves in two halves of four.  Both halves have the same queries and heads and
// each takes every other page of the keys, with LDS stages of its own; at the end the second half
// hands its sums and softmax statistics to the first through LDS.  The longest tiles, which set
// the kernel's time when a prompt gives each CU only a tile or two, then take half as long.
// (up to head size 128 two waves share a SIMD's registers, 256 each; the sums and operands of a
// larger head need more, and a wave then has the SIMD to itself)
template <int D, int HALVES>
__global__ __launch_bounds__(256 * HALVES) __attribute__((amdgpu_waves_per_eu(D <= 128 ? 2 : 1))) void attn_prefill_mfma_kernel(
    AttnArgs a, int HB, int tile_tokens, int n_tiles, int n_cus) {
    constexpr int LOADS = D / 32;                     // KB of a page's K (and of its V^T) that a wave brings in
    constexpr int STAGE = 2 * PAGE_TOKENS * D;        // K tile + V^T tile, in bf16
    extern __shared__ __attribute__((aligned(1024))) bf16_t lds_all[];    // two stages for each half
    const int half = __builtin_amdgcn_readfirstlane(threadIdx.x / 256);
    bf16_t* lds = lds_all + half * (2 * STAGE);
    const int tid = threadIdx.x % 256, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // (within the half)
    const int l32 = lane % 32, h = lane / 32;
    const int R = a.H / a.G;
    const int head_chunks = (R + HB - 1) / HB;
    // The host lists the tiles with the fewest keys first.  Work items (tile, group of heads) are
    // handed out longest first, in rounds of one workgroup per CU, and every other round runs
    // backwards: the workgroups that share a CU from the start (a CU holds two) then have a long
    // and a short tile, where the same order in every round would pair the longest with each other.
    const int per_tile = a.G * head_chunks;
    const int total = n_tiles * per_tile;
    // (with HALVES = 2 a CU holds one workgroup at a time and takes the next when it is done:
    // longest first as it is)
    const int round0 = (int)(blockIdx.x / n_cus) * n_cus, in_round = blockIdx.x - round0;
    const int round_size = min(n_cus, total - round0);
    const int item = HALVES == 2 ? (int)blockIdx.x
                                 : round0 + (((blockIdx.x / n_cus) & 1) ? round_size - 1 - in_round : in_round);
    const int tile_id = n_tiles - 1 - item / per_tile;
    const int which = item % per_tile;
    const int seq = a.tile_seq[tile_id], q0 = a.tile_q0[tile_id];
    const int g = which / head_chunks, chunk = which % head_chunks;
    const int head_local = chunk * HB + wave % HB;
    const int tb = wave / HB;
    const int nnew = a.seq_nnew[seq], pos0 = a.seq_pos0[seq];
    const int w_first = q0 + 32 * tb;
    const bool w_active = head_local < R && w_first < nnew;
    const int head = g * R + (head_local < R ? head_local : 0);
    const int qi = w_first + l32;
    const bool q_ok = w_active && qi < nnew;
    const int qpos = pos0 + qi;
    const size_t tok = (size_t)a.cu_seqlens[seq] + (q_ok ? qi : 0);

    const int b_qfirst = pos0 + q0, b_qlast = pos0 + min(q0 + tile_tokens, nnew) - 1;
    const int page_lo = (a.window > 0 ? max(0, b_qfirst - a.window + 1) : 0) / PAGE_TOKENS;
    const int page_hi = b_qlast / PAGE_TOKENS + 1;
    const int w_qfirst = pos0 + w_first, w_qlast = pos0 + min(w_first + 32, nnew) - 1;
    const int w_page_lo = (a.window > 0 ? max(0, w_qfirst - a.window + 1) : 0) / PAGE_TOKENS;
    const int w_page_hi = w_active ? w_qlast / PAGE_TOKENS + 1 : 0;

    bf16x8 Qf[D / 16];
    f32x16 O[D / 32];
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) O[dt][e] = 0.f;
    float m_run = NEG_BIG, l_run = 0.f;
    const float scale2 = a.scale * LOG2E;
    const int32_t* pt = a.page_table + (size_t)a.seq_slot[seq] * a.max_pages;
    const size_t page_elems = (size_t)a.G * PAGE_TOKENS * D;

    // A page's K and V^T go from the cache straight into LDS: as they lie in the cache they are in
    // the order of the MFMA operands, so a wave copies whole kilobytes (wave w of a half the KB
    // w, w + 4, ..).  Where a page lies is asked a round ahead of its loads, which would otherwise
    // wait for it.
    auto place_of = [&](int page) { return __builtin_amdgcn_readfirstlane(pt[page % a.ring_pages]); };
    const unsigned lds_wave = __builtin_amdgcn_readfirstlane(
        (unsigned)(size_t)(__attribute__((address_space(3))) bf16_t*)lds + wave * 1024);
    const unsigned lane_bytes = lane * 16;
    auto fetch = [&](int stage, int place) {
        const size_t base = (size_t)place * page_elems + (size_t)g * PAGE_TOKENS * D;
        const char* kp = (const char*)((const bf16_t*)a.k_pages + base) + wave * 1024;
        const char* vp = (const char*)((const bf16_t*)a.v_pages + base) + wave * 1024;
        const unsigned to = lds_wave + stage * (STAGE * 2);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) load_16_bytes_to_lds(lane_bytes, same_in_every_lane(kp + i * 4096), to + i * 4096);
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            load_16_bytes_to_lds(lane_bytes, same_in_every_lane(vp + i * 4096), to + PAGE_TOKENS * D * 2 + i * 4096);
    };
    // What a wave has brought in is in LDS; before the others may read it, the values of keys past
    // the sequence's end, which may hold anything, are zeroed (their probabilities are zero, but
    // zero times anything is not).  Only a tile's last page has such keys.
    auto landed = [&](int stage, int page) {
        wait_for_loads<0>();
        const int n_keys = b_qlast - page * PAGE_TOKENS + 1;
        if (n_keys < PAGE_TOKENS) {
            bf16_t* Vs = lds + stage * STAGE + PAGE_TOKENS * D;
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int idx = tid + 256 * i;
                // chunk idx of V^T holds keys 32*tile + 16*step + 8*half .. + 8 (see v_page_offset)
                const int key0 = 32 * (idx / (128 * (D / 32))) + 16 * ((idx / 64) % 2) + 8 * ((idx % 64) / 32);
                bf16x8 v = *(const bf16x8*)(Vs + (size_t)idx * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (key0 + e < n_keys) ? v[e] : (__bf16)0.0f;
                *(bf16x8*)(Vs + (size_t)idx * 8) = v;
            }
        }
        __syncthreads();
    };
    auto operands = [&](int stage) {
        const bf16_t* Ks = lds + stage * STAGE;
        const bf16_t* Vs = Ks + PAGE_TOKENS * D;
        return std::make_pair(
            [=](int t, int s) { return *(const bf16x8*)(Ks + ((t * (D / 16) + s) * 64 + lane) * 8); },
            [=](int dt, int t, int ks) { return *(const bf16x8*)(Vs + (((t * (D / 32) + dt) * 2 + ks) * 64 + lane) * 8); });
    };
    // a page wholly before the tile's first query: every wave attends to all of it (rows
    // without a query are never stored, whatever they hold)
    auto compute_plain = [&](int stage, int page) {
        const auto op = operands(stage);
        attend_page<D, false>(Qf, O, m_run, l_run, page * PAGE_TOKENS, qpos, q_ok, a.window, scale2, h, op.first, op.second);
    };
    auto compute = [&](int stage, int page) {
        if (page < w_page_lo || page >= w_page_hi) return;
        const auto op = operands(stage);
        // a page wholly before the wave's first query needs no mask
        if (a.window <= 0 && page * PAGE_TOKENS + PAGE_TOKENS - 1 <= w_qfirst)
            attend_page<D, false>(Qf, O, m_run, l_run, page * PAGE_TOKENS, qpos, q_ok, a.window, scale2, h, op.first, op.second);
        else
            attend_page<D, true>(Qf, O, m_run, l_run, page * PAGE_TOKENS, qpos, q_ok, a.window, scale2, h, op.first, op.second);
    };

    // a half's pages: page_lo + half, then every HALVES-th; both halves go round the loop alike
    const int n_rounds = (page_hi - page_lo + HALVES - 1) / HALVES;
    auto page_of = [&](int round) { return page_lo + HALVES * round + half; };
    // (A half whose turn has no page left brings in the tile's last page again and attends to
    // nothing: loads without conditions around them keep the waits for them apart from the matrix
    // products.)
    fetch(0, place_of(min(page_of(0), page_hi - 1)));
    int next_place = place_of(min(page_of(1), page_hi - 1));
    // the queries, while the first page is on its way
    if (a.qkv) {        // the float rows of the qkv product: rotated here, no rotated copy of q in memory
        rotated_q<D>(a, a.qkv + tok * (size_t)(a.H + 2 * a.G) * D + (size_t)head * D, qpos, h, q_ok, Qf);
    } else {
        const bf16_t* qp = (const bf16_t*)a.q + tok * a.H * D + (size_t)head * D + 8 * h;
#pragma unroll
        for (int s = 0; s < D / 16; ++s) Qf[s] = q_ok ? ldg8(qp + 16 * s) : zero8();
    }
    landed(0, min(page_of(0), page_hi - 1));
    int cur = 0, round = 0;
    // The rounds whose pages lie wholly before the tile's first query, most of a long prompt's,
    // have a loop of their own with one path through it: in the general loop below, where a wave
    // may skip a page or mask it, the compiler moves all of O^T between registers twice a page.
    const int plain_rounds = a.window > 0 ? 0 : min(n_rounds - 1, max(0, (b_qfirst / PAGE_TOKENS - page_lo) / HALVES));
    for (; round < plain_rounds; ++round) {
        const int next = min(page_of(round + 1), page_hi - 1);
        fetch(cur ^ 1, next_place);               // in flight while this page is attended to
        next_place = place_of(min(page_of(round + 2), page_hi - 1));
        __builtin_amdgcn_sched_barrier(0);
        compute_plain(cur, page_of(round));
        __builtin_amdgcn_sched_barrier(0);
        landed(cur ^ 1, next);
        cur ^= 1;
    }
    for (; round + 1 < n_rounds; ++round) {
        const int next = min(page_of(round + 1), page_hi - 1);
        fetch(cur ^ 1, next_place);
        next_place = place_of(min(page_of(round + 2), page_hi - 1));
        __builtin_amdgcn_sched_barrier(0);
        compute(cur, page_of(round));
        __builtin_amdgcn_sched_barrier(0);
        landed(cur ^ 1, next);
        cur ^= 1;
    }
    compute(cur, page_of(n_rounds - 1));          // (past the tile's pages: nothing)

    if (HALVES == 2) {
        // The second half's O^T, reference point and sum of each lane go to the first half's lane
        // of the same place through LDS (the stages are read out by now): value v of all lanes of a
        // wave side by side.
        __syncthreads();
        float* hand = (float*)lds_all + (size_t)wave * (D / 32 * 16 + 2) * WAVE + lane;
        if (half == 1) {
#pragma unroll
            for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) hand[(dt * 16 + e) * WAVE] = O[dt][e];
            hand[(D / 32 * 16) * WAVE] = m_run;
            hand[(D / 32 * 16 + 1) * WAVE] = l_run;
        }
        __syncthreads();
        if (half == 1) return;
        const float m_other = hand[(D / 32 * 16) * WAVE], l_other = hand[(D / 32 * 16 + 1) * WAVE];
        const float m_both = fmaxf(m_run, m_other);
        const float mine = exp2_flushing(m_run - m_both), other = exp2_flushing(m_other - m_both);
        l_run = l_run * mine + l_other * other;
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) O[dt][e] = O[dt][e] * mine + hand[(dt * 16 + e) * WAVE] * other;
    }
    if (!q_ok) return;
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    bf16_t* o = (bf16_t*)a.out + tok * a.H * D + (size_t)head * D;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            bf16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = to_bf16(O[dt][4 * q4 + e] * inv);
            *(bf16x4*)(o + 32 * dt + 8 * q4 + 4 * h) = v;
        }
}

// =============================================================================================
// One new token per sequence.  A workgroup takes a chunk of pages of one sequence and one KV
// group; its waves take the chunk's tiles of 32 keys in turn, each asking for a whole tile (keys
// and values) before it waits for any of it.  What a workgroup needs to find its pages comes in
// one 32-byte entry of the work list, so that only two trips to memory lie between the launch
// and the first MFMA.  Eight waves give a short step for a few sequences; with many sequences
// four waves, two workgroups a CU, move more bytes.
// With a.qkv set the rotation and the cache write of the new token happen here too: q is rotated
// on its way into the MFMA operands; the workgroups of a sequence's last chunk rotate the new key,
// round key and value to bfloat16 as the cache holds them, put them into the merge below as one
// more partial result (score, weight 1, value), and one of them writes them to the cache for
// later steps.  The cache row of the new token is not read in this step.
// single accesses that every workgroup of the GPU sees alike
__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int D, int DEC_WAVES>
__global__ __launch_bounds__(DEC_WAVES * 64) __attribute__((amdgpu_waves_per_eu(D <= 128 ? 2 : 1))) void attn_decode_mfma_kernel(AttnArgs a) {
    extern __shared__ float mrg[];       // [DEC_WAVES + 1][Rc][D + 2], then the new key and value [2][D]
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int l32 = lane % 32, h = lane / 32;
    const int R = a.H / a.G;
    const int chunks = (R + 31) / 32;
    DecodeWork work;
    int which;
    if (!decode_work(a, a.G * chunks, work, which)) return;
    const int seq = work.seq, split = work.split;
    const int g = which / chunks, chunk = which % chunks;
    const int Rc = min(32, R - chunk * 32);
    const bool q_ok = l32 < Rc;
    const int head = g * R + chunk * 32 + (q_ok ? l32 : 0);
    const size_t tok = (size_t)seq;
    const int qpos = work.qpos;
    const bool fused = a.qkv != nullptr;
    const bool takes_new = fused && split == work.n_chunks - 1;       // this chunk ends with the new token
    const int key_max = fused ? qpos - 1 : qpos;                       // the last key read from the cache
    float* knew = mrg + (size_t)(DEC_WAVES + 1) * Rc * (D + 2);
    float* vnew = knew + D;

    const int page_lo = work.page_lo, page_hi = work.page_hi;
    // k-step s of a lane covers d = 16s + 8h .. +8: the two halves of a wave read 32 adjacent bytes of a key
    bf16x8 Qf[D / 16];
    if (fused) {
        const float* row = a.qkv + tok * (size_t)(a.H + 2 * a.G) * D;
        rotated_q<D>(a, row + (size_t)head * D, qpos, h, q_ok, Qf);
        if (takes_new) {
            const float* krow = row + (size_t)(a.H + g) * D;
            const float* vrow = row + (size_t)(a.H + a.G + g) * D;
            if (tid < D / 2) {
                const int i0 = a.rope_style == 0 ? 2 * tid : tid, i1 = a.rope_style == 0 ? 2 * tid + 1 : tid + D / 2;
                const float x0 = krow[i0], x1 = krow[i1];
                float y0 = x0, y1 = x1;
                if (a.cos_t) {
                    const float cc = a.cos_t[(size_t)qpos * (D / 2) + tid], ss = a.sin_t[(size_t)qpos * (D / 2) + tid];
                    y0 = x0 * cc - x1 * ss;
                    y1 = x0 * ss + x1 * cc;
                }
                knew[i0] = (float)to_bf16(y0);
                knew[i1] = (float)to_bf16(y1);
            }
            for (int i = tid; i < D; i += DEC_WAVES * 64) vnew[i] = (float)to_bf16(vrow[i]);
        }
    } else {
        const bf16_t* qp = (const bf16_t*)a.q + tok * a.H * D + (size_t)head * D + 8 * h;
#pragma unroll
        for (int s = 0; s < D / 16; ++s) Qf[s] = q_ok ? ldg8(qp + 16 * s) : zero8();
    }
    f32x16 O[D / 32];
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) O[dt][e] = 0.f;
    float m_run = NEG_BIG, l_run = 0.f;
    const float scale2 = a.scale * LOG2E;
    const int32_t* pt = a.page_table + (size_t)work.slot * a.max_pages;
    const size_t page_elems = (size_t)a.G * PAGE_TOKENS * D;

    // tile tt of the chunk: keys 32*tt .. 32*tt+31 counted from the chunk's first page
    const int n_tiles = 2 * (page_hi - page_lo);
    auto page_of_tile = [&](int tt) {                       // the first eight tiles' pages came with the entry
        if (tt >= n_tiles) return 0;
        if (tt >= 8) return pt[(page_lo + tt / 2) % a.ring_pages];
        return tt < 2 ? work.phys[0] : tt < 4 ? work.phys[1] : tt < 6 ? work.phys[2] : work.phys[3];
    };
    // whether anything of tile tt is visible (if not, nothing of a later one is either)
    auto visible = [&](int tt) { return tt < n_tiles && (page_lo + tt / 2) * PAGE_TOKENS + 32 * (tt & 1) <= key_max; };
    // tile t of the group's part of a page: 32 * D elements of K, then of V^T, as operands
    auto tile_offset = [&](int tt, int phys) {
        return (size_t)phys * page_elems + (size_t)g * PAGE_TOKENS * D + (size_t)(tt & 1) * 32 * D + lane * 8;
    };
    // A wave takes tiles wave, wave + DEC_WAVES, ..  The keys of its next tile are asked for before
    // it attends to this one, and this tile's values when its keys are already there: the scores and
    // the softmax run while the values are on their way.  The page of the tile after the next is
    // looked up a round ahead of its loads.
    bf16x8 Kf[D / 16], Kn[D / 16], Vf[D / 32][2];
    const bool once = chunks == 1;        // all heads of the group are here: nobody else reads these keys and values
    int tt = wave;
    bool have = visible(tt);
    int phys = page_of_tile(tt), phys_next = page_of_tile(tt + DEC_WAVES);
    if (have) {
        load_tile_chunks(Kf, (const bf16_t*)a.k_pages + tile_offset(tt, phys), once);
    }
    while (have) {
        const int key0 = (page_lo + tt / 2) * PAGE_TOKENS + 32 * (tt & 1);
        const int n_keys = key_max - key0 + 1;               // >= 1; keys past it are not this sequence's, or not written yet
        load_tile_chunks((bf16x8(&)[D / 16])Vf, (const bf16_t*)a.v_pages + tile_offset(tt, phys), once);
        const int tn = tt + DEC_WAVES;
        const bool have_next = visible(tn);
        const int phys_after = page_of_tile(tn + DEC_WAVES);
        if (have_next) {
            load_tile_chunks(Kn, (const bf16_t*)a.k_pages + tile_offset(tn, phys_next), once);
        }
        if (n_keys < 32) {                                   // keys past the end may hold anything
#pragma unroll
            for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const int k = 16 * ks + 8 * h;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k + e >= n_keys) Vf[dt][ks][e] = (__bf16)0.0f;
                }
        }
        attend_tile<D>(Qf, Kf, Vf, O, m_run, l_run, key0, key_max, qpos, q_ok, a.window, scale2, h);
#pragma unroll
        for (int s = 0; s < D / 16; ++s) Kf[s] = Kn[s];
        tt = tn;
        have = have_next;
        phys = phys_next;
        phys_next = phys_after;
    }
    // merge the waves
    float* mine = mrg + (size_t)wave * Rc * (D + 2);
    if (q_ok) {
        float* row = mine + (size_t)l32 * (D + 2);
        if (h == 0) {
            row[0] = m_run;
            row[1] = l_run;
        }
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) row[2 + 32 * dt + 8 * (e / 4) + 4 * h + e % 4] = O[dt][e];
    }
    __syncthreads();
    if (takes_new) {
        // the new token as the partial result of one more wave: its score with every head of this
        // workgroup, weight 1, its value
        if (wave == 0 && q_ok) {
            float dot = 0.f;
#pragma unroll
            for (int s = 0; s < D / 16; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) dot += (float)Qf[s][e] * knew[16 * s + 8 * h + e];
            dot += __shfl_xor(dot, 32, WAVE);
            if (h == 0) {
                float* row = mrg + ((size_t)DEC_WAVES * Rc + l32) * (D + 2);
                row[0] = dot * scale2;
                row[1] = 1.0f;
            }
        }
        if (chunk == 0 && tid < D) {                        // one workgroup of the group writes the cache
            const size_t base = (size_t)a.tok_page[seq] * page_elems + (size_t)g * PAGE_TOKENS * D;
            const int in_page = qpos % PAGE_TOKENS;
            ((bf16_t*)a.k_pages)[base + k_page_offset(in_page, tid, D, true)] = f32_to_bf16_bits(knew[tid]);
            ((bf16_t*)a.v_pages)[base + v_page_offset(tid, in_page, D, true)] = f32_to_bf16_bits(vnew[tid]);
        }
        __syncthreads();
    }
    const int n_parts = takes_new ? DEC_WAVES + 1 : DEC_WAVES;
    for (int idx = tid; idx < Rc * D; idx += DEC_WAVES * 64) {
        const int q = idx / D, dcol = idx % D;
        float M = NEG_BIG;
        for (int w = 0; w < n_parts; ++w) M = fmaxf(M, mrg[((size_t)w * Rc + q) * (D + 2)]);
        float L = 0.f, acc = 0.f;
        for (int w = 0; w < n_parts; ++w) {
            const float* row = mrg + ((size_t)w * Rc + q) * (D + 2);
            const float f = exp2f(row[0] - M);
            L += f * row[1];
            acc += f * (w < DEC_WAVES ? row[2 + dcol] : vnew[dcol]);
        }
        const int hq = g * R + chunk * 32 + q;
        if (work.n_chunks > 1) {
            float* po = a.partial + (((size_t)seq * a.H + hq) * a.max_splits + split) * (D + 2);
            if (a.chunks_done) {        // read back by another workgroup of this launch
                if (dcol == 0) {
                    store_agent(po, M * LN2);
                    store_agent(po + 1, L);
                }
                store_agent(po + 2 + dcol, acc);
            } else {
                if (dcol == 0) {
                    po[0] = M * LN2;        // the merge kernel works with natural exponents
                    po[1] = L;
                }
                po[2 + dcol] = acc;
            }
        } else {
            ((bf16_t*)a.out)[tok * a.H * D + (size_t)hq * D + dcol] = f32_to_bf16_bits(L > 0.f ? acc / L : 0.f);
        }
    }
    if (work.n_chunks <= 1 || a.chunks_done == nullptr) return;       // (uniform over the workgroup)
    // The chunks of a sequence finish in any order.  Each workgroup counts itself once its partial
    // results have arrived in memory; the one that counts last reads them all back and writes the
    // output, chunk by chunk in their order, so the sum does not depend on who it was.  The
    // partial results are written and read as single accesses that are coherent over the whole GPU
    // (they pass the L2 of the chiplet): a fence of that scope would write back and invalidate
    // the whole L2 in every workgroup, which costs far more than the merge kernel it replaces.
    __shared__ int i_am_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this thread's stores have been acknowledged
    __syncthreads();
    int32_t* counter = a.chunks_done + (size_t)seq * (a.G * chunks) + which;
    if (tid == 0)
        i_am_last = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == work.n_chunks - 1;
    __syncthreads();
    if (!i_am_last) return;
    const int n = work.n_chunks;
    for (int idx = tid; idx < Rc * D; idx += DEC_WAVES * 64) {
        const int q = idx / D, dcol = idx % D;
        const int hq = g * R + chunk * 32 + q;
        const float* p = a.partial + ((size_t)seq * a.H + hq) * a.max_splits * (D + 2);
        float M = NEG_BIG, L = 0.f, acc = 0.f;
        for (int i0 = 0; i0 < n; i0 += 8) {             // eight chunks are asked for at a time
            float st[8], li[8], col[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float* pe = p + (size_t)min(i0 + e, n - 1) * (D + 2);
                st[e] = load_agent(pe);
                li[e] = load_agent(pe + 1);
                col[e] = load_agent(pe + 2 + dcol);
            }
            float m_new = M;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (i0 + e < n) m_new = fmaxf(m_new, st[e]);
            const float keep = expf(M - m_new);
            L *= keep;
            acc *= keep;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (i0 + e < n) {
                    const float f = expf(st[e] - m_new);
                    L += f * li[e];
                    acc += f * col[e];
                }
            M = m_new;
        }
        ((bf16_t*)a.out)[tok * a.H * D + (size_t)hq * D + dcol] = f32_to_bf16_bits(L > 0.f ? acc / L : 0.f);
    }
    if (tid == 0) *counter = 0;          // as the next launch expects it
}

// =============================================================================================
extern "C" int picolm_attn_mfma_takes(int d);
static int check_sizes(const char* who, int H, int G, int d, int max_pages, int ring_pages) {
    PICOLM_REQUIRE(H > 0 && G > 0 && H % G == 0, "%s: %d heads do not split over %d groups", who, H, G);
    PICOLM_REQUIRE(picolm_attn_mfma_takes(d), "%s: head size %d is no multiple of 32 up to 256", who, d);
    PICOLM_REQUIRE(max_pages > 0 && ring_pages > 0 && ring_pages <= max_pages,
                   "%s: bad page table geometry max_pages=%d ring_pages=%d", who, max_pages, ring_pages);
    return 0;
}

extern "C" int picolm_attn_mfma_takes(int d) { return d >= 32 && d <= 256 && d % 32 == 0; }

// LDS of a decode workgroup of `waves` waves: the waves' partial results and the new token's, then
// the new key and value
static size_t decode_lds_bytes(int R, int d, int waves) { return sizeof(float) * ((waves + 1) * (size_t)min(R, 32) * (d + 2) + 2 * d); }
static const size_t LDS_LIMIT = 160 * 1024;

// Whether the matrix-core kernels take this shape: the head size, and a decode workgroup's partial
// results (32 query heads of a group at most, each of d + 2 floats, from four waves) within LDS.
extern "C" int picolm_attn_mfma_fits(int H, int G, int d) {
    if (!picolm_attn_mfma_takes(d) || G <= 0 || H % G) return 0;
    return decode_lds_bytes(H / G, d, 4) <= LDS_LIMIT;
}

// heads of a group that share a workgroup, and the new tokens one workgroup covers
extern "C" int picolm_attn_prefill_mfma_heads(int H, int G) {
    const int R = H / G;
    return R >= 3 ? 4 : (R == 2 ? 2 : 1);
}
extern "C" int picolm_attn_prefill_mfma_tile_tokens(int H, int G) {
    return 32 * (4 / picolm_attn_prefill_mfma_heads(H, G));
}

static int launch_prefill_mfma(AttnArgs a, int n_tiles, hipStream_t stream) {
    const int H = a.H, G = a.G, d = a.d;
    const int HB = picolm_attn_prefill_mfma_heads(H, G);
    const int tile_tokens = 32 * (4 / HB);
    const int head_chunks = ceil_div(H / G, HB);
    PICOLM_REQUIRE((int64_t)n_tiles * G * head_chunks < (1ll << 31), "attn_prefill_mfma: too many workgroups");
    static int n_cus = 0;
    if (n_cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        PICOLM_REQUIRE(hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess,
                       "attn_prefill_mfma: cannot read the device's properties");
        n_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 1;
    }
    // Up to a tile for each of a CU's two places the longest tile sets the time, and eight waves
    // that share its pages halve it (measured at head size 128: 43 -> 33 us for 1,024 tokens, 85 -> 75
    // for 2,048); with more tiles the CUs even out by themselves and two independent workgroups a CU
    // overlap better than eight waves in step (219 against 243 us for 4,096 tokens).
    // (two halves have two stages of K and V^T each: head sizes above 128 would not fit LDS)
    const int halves = (int64_t)n_tiles * G * head_chunks <= 2 * (int64_t)n_cus && d <= 128 ? 2 : 1;
    dim3 grid(n_tiles * G * head_chunks), block(256 * halves);
    const size_t lds = halves * 2 * 2 * (size_t)PAGE_TOKENS * d * sizeof(bf16_t);       // two stages of K and V^T a half
#define PREFILL_LAUNCH(D, HALVES)                                                                             \
    {                                                                                                         \
        static size_t raised = 48 * 1024;                                                                     \
        if (lds > raised) {                                                                                   \
            hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_mfma_kernel<D, HALVES>,              \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
            PICOLM_REQUIRE(e == hipSuccess, "attn_prefill_mfma: cannot raise the LDS limit: %s",              \
                           hipGetErrorString(e));                                                             \
            raised = lds;                                                                                     \
        }                                                                                                     \
        attn_prefill_mfma_kernel<D, HALVES><<<grid, block, lds, stream>>>(a, HB, tile_tokens, n_tiles, n_cus); \
    }
#define PREFILL_BOTH(D)                   \
    if (halves == 2) PREFILL_LAUNCH(D, 2) \
    else PREFILL_LAUNCH(D, 1)
    switch (d) {
        case 32: PREFILL_BOTH(32) break;
        case 64: PREFILL_BOTH(64) break;
        case 96: PREFILL_BOTH(96) break;
        case 128: PREFILL_BOTH(128) break;
        case 160: PREFILL_LAUNCH(160, 1) break;
        case 192: PREFILL_LAUNCH(192, 1) break;
        case 224: PREFILL_LAUNCH(224, 1) break;
        default: PREFILL_LAUNCH(256, 1) break;
    }
#undef PREFILL_BOTH
#undef PREFILL_LAUNCH
    PICOLM_LAUNCH_CHECK("attn_prefill_mfma");
    return 0;
}

extern "C" int picolm_attn_prefill_mfma(const void* q, const void* k_pages, const void* v_pages, void* out,
                                        const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                                        const int32_t* seq_slot, const int32_t* seq_pos0,
                                        const int32_t* seq_nnew, const int32_t* cu_seqlens,
                                        const int32_t* page_table, int max_pages, int ring_pages, int H, int G,
                                        int d, int window, float scale, hipStream_t stream) {
    if (check_sizes("attn_prefill_mfma", H, G, d, max_pages, ring_pages)) return -1;
    if (n_tiles <= 0) return 0;
    AttnArgs a = {q, k_pages, v_pages, out, nullptr, tile_seq, tile_q0, seq_slot, seq_pos0, seq_nnew,
                  cu_seqlens, page_table, max_pages, ring_pages, H, G, d, window, scale, 0, nullptr, 0, 1,
                  nullptr, nullptr, nullptr, nullptr, 0};
    return launch_prefill_mfma(a, n_tiles, stream);
}

// Whether a prefill step of T tokens should let the attention kernel rotate q itself
// (picolm_kv_store_tiles + picolm_attn_prefill_rope_mfma) rather than read a rotated copy
// (picolm_rope_kv_store + picolm_attn_prefill_mfma).  Without the copy a layer of 2,048 tokens
// takes 84 us for the two kernels instead of 94, one of 8,192 tokens 4 % less; but a short prompt
// has few workgroups, each of which then rotates its queries before it can start, where the
// rotation kernel spreads that over the GPU: 24 us against 17 at 128 tokens, 32 against 30 at 512.
extern "C" int picolm_attn_prefill_rotates_q(int T) { return T >= 1024; }

// The same with the queries taken from the float rows qkv[T][(H+2G)*d] of the step and rotated on
// their way into the kernel (cos_t, sin_t [positions][d/2], both null: no rotation; style as in
// picolm_rope_kv_store): no rotated copy of q is written or read.  The keys and values of the
// step's tokens must be in the cache already (picolm_rope_kv_store with q_out null).
extern "C" int picolm_attn_prefill_rope_mfma(const float* qkv, const void* k_pages, const void* v_pages, void* out,
                                             const int32_t* tile_seq, const int32_t* tile_q0, int n_tiles,
                                             const int32_t* seq_slot, const int32_t* seq_pos0,
                                             const int32_t* seq_nnew, const int32_t* cu_seqlens,
                                             const int32_t* page_table, int max_pages, int ring_pages, int H, int G,
                                             int d, int window, float scale, const float* cos_t, const float* sin_t,
                                             int style, hipStream_t stream) {
    if (check_sizes("attn_prefill_rope_mfma", H, G, d, max_pages, ring_pages)) return -1;
    PICOLM_REQUIRE(qkv != nullptr && ((uintptr_t)qkv & 15) == 0, "attn_prefill_rope_mfma: the qkv rows must be 16-byte aligned");
    PICOLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attn_prefill_rope_mfma: need both tables or none");
    PICOLM_REQUIRE(style == 0 || style == 1, "attn_prefill_rope_mfma: unknown pairing %d", style);
    if (n_tiles <= 0) return 0;
    AttnArgs a = {nullptr, k_pages, v_pages, out, nullptr, tile_seq, tile_q0, seq_slot, seq_pos0, seq_nnew,
                  cu_seqlens, page_table, max_pages, ring_pages, H, G, d, window, scale, 0, nullptr, 0, 1,
                  qkv, cos_t, sin_t, nullptr, style};
    return launch_prefill_mfma(a, n_tiles, stream);
}

int check_decode_chunks(const char* who, const float* partial, const int32_t* chunk_list, int n_chunks,
                        int pages_per_chunk, int max_splits);
int picolm_attn_merge_launch(const AttnArgs& a, int dt, int n_seq, hipStream_t stream);

// waves of a decode workgroup: eight while every sequence's workgroups are at most two a CU of
// 256 (a sequence's pages are a shorter chain for each wave); beyond that four waves move more
// bytes.  Measured, eight against four waves a step: 256 workgroups 4.59 against 4.61 ms (8 KV
// groups of head size 128, batch 32) and 1.41 against 1.53 (head size 64); 384: 5.16 against
// 5.37; 512: 5.74 against 5.83, 1.78 against 1.80, and 3.98 against 3.96 (32 KV groups, batch
// 16); 1,024: 8.77 against 8.64; 2,048: 8.37 against 7.81.
extern "C" int picolm_attn_decode_mfma_waves(int n_seq, int H, int G) {
    const int chunks = ceil_div(H / (G > 0 ? G : 1), 32);
    return (int64_t)n_seq * G * chunks > 512 ? 4 : 8;
}

static int launch_decode_mfma(const AttnArgs& a, int n_seq, int n_chunks, hipStream_t stream) {
    const int R = a.H / a.G, chunks = ceil_div(R, 32), d = a.d;
    PICOLM_REQUIRE((int64_t)n_chunks * a.G * chunks < (1ll << 31), "attn_decode_mfma: %d chunks of %d workgroups exceed the grid", n_chunks, a.G * chunks);
    int waves = picolm_attn_decode_mfma_waves(n_seq, a.H, a.G);
    // (a head above 128 needs a SIMD's registers for one wave; many wide heads a group: the partial
    // results of eight waves do not fit LDS)
    if (d > 128 || decode_lds_bytes(R, d, waves) > LDS_LIMIT) waves = 4;
    PICOLM_REQUIRE(decode_lds_bytes(R, d, waves) <= LDS_LIMIT, "attn_decode_mfma: %d heads of size %d a group need more LDS than a CU has", R, d);
    dim3 grid(n_chunks * a.G * chunks), block(waves * 64);
    const size_t lds = decode_lds_bytes(R, d, waves);
#define DEC_LAUNCH(D, W)                                                                                    \
    {                                                                                                       \
        static size_t raised = 48 * 1024;                                                                   \
        if (lds > raised) {                                                                                 \
            hipError_t e = hipFuncSetAttribute((const void*)attn_decode_mfma_kernel<D, W>,                  \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);       \
            PICOLM_REQUIRE(e == hipSuccess, "attn_decode_mfma: cannot raise the LDS limit: %s",             \
                           hipGetErrorString(e));                                                           \
            raised = lds;                                                                                   \
        }                                                                                                   \
        attn_decode_mfma_kernel<D, W><<<grid, block, lds, stream>>>(a);                                     \
    }
#define DEC_BOTH(D)                  \
    if (waves == 4) DEC_LAUNCH(D, 4) \
    else DEC_LAUNCH(D, 8)
    switch (d) {
        case 32: DEC_BOTH(32) break;
        case 64: DEC_BOTH(64) break;
        case 96: DEC_BOTH(96) break;
        case 128: DEC_BOTH(128) break;
        case 160: DEC_LAUNCH(160, 4) break;
        case 192: DEC_LAUNCH(192, 4) break;
        case 224: DEC_LAUNCH(224, 4) break;
        default: DEC_LAUNCH(256, 4) break;
    }
#undef DEC_BOTH
#undef DEC_LAUNCH
    PICOLM_LAUNCH_CHECK("attn_decode_mfma");
    return a.max_splits > 1 && !a.chunks_done ? picolm_attn_merge_launch(a, PICOLM_BF16, n_seq, stream) : 0;
}

extern "C" int picolm_attn_decode_mfma(const void* q, const void* k_pages, const void* v_pages, void* out,
                                       float* partial, int n_seq, const int32_t* chunk_list, int n_chunks,
                                       int pages_per_chunk, int max_splits, const int32_t* seq_pos0,
                                       const int32_t* page_table, int max_pages, int ring_pages, int H, int G,
                                       int d, int window, float scale, int32_t* chunks_done, hipStream_t stream) {
    if (check_sizes("attn_decode_mfma", H, G, d, max_pages, ring_pages)) return -1;
    if (check_decode_chunks("attn_decode_mfma", partial, chunk_list, n_chunks, pages_per_chunk, max_splits)) return -1;
    if (n_seq <= 0 || n_chunks <= 0) return 0;
    AttnArgs a = {q, k_pages, v_pages, out, partial, nullptr, nullptr, nullptr, seq_pos0, nullptr, nullptr,
                  page_table, max_pages, ring_pages, H, G, d, window, scale, 1, chunk_list, pages_per_chunk, max_splits,
                  nullptr, nullptr, nullptr, nullptr, 0, chunks_done};
    return launch_decode_mfma(a, n_seq, n_chunks, stream);
}

// The decode step's rotation, cache write and attention in one launch: q, k, v of the new tokens
// come as the float rows qkv[n_seq][(H+2G)*d]; tok_page[i] is the physical page that takes
// sequence i's new key and value.  cos_t, sin_t [positions][d/2] or both null for no rotation.
extern "C" int picolm_attn_decode_rope_mfma(const float* qkv, void* k_pages, void* v_pages, void* out,
                                            float* partial, int n_seq, const int32_t* chunk_list, int n_chunks,
                                            int pages_per_chunk, int max_splits, const int32_t* seq_pos0,
                                            const int32_t* page_table, int max_pages, int ring_pages, int H,
                                            int G, int d, int window, float scale, const float* cos_t,
                                            const float* sin_t, int style, const int32_t* tok_page,
                                            int32_t* chunks_done, hipStream_t stream) {
    if (check_sizes("attn_decode_rope_mfma", H, G, d, max_pages, ring_pages)) return -1;
    if (check_decode_chunks("attn_decode_rope_mfma", partial, chunk_list, n_chunks, pages_per_chunk, max_splits)) return -1;
    PICOLM_REQUIRE(qkv && tok_page, "attn_decode_rope_mfma: needs the qkv rows and every token's page");
    PICOLM_REQUIRE(((uintptr_t)qkv & 15) == 0 && ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0,
                   "attn_decode_rope_mfma: qkv and the tables must be 16-byte aligned");
    PICOLM_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attn_decode_rope_mfma: need both tables or none");
    PICOLM_REQUIRE(style == 0 || style == 1, "attn_decode_rope_mfma: unknown pairing %d", style);
    if (n_seq <= 0 || n_chunks <= 0) return 0;
    AttnArgs a = {nullptr, k_pages, v_pages, out, partial, nullptr, nullptr, nullptr, seq_pos0, nullptr, nullptr,
                  page_table, max_pages, ring_pages, H, G, d, window, scale, 1, chunk_list, pages_per_chunk, max_splits,
                  qkv, cos_t, sin_t, tok_page, style, chunks_done};
    return launch_decode_mfma(a, n_seq, n_chunks, stream);
}
