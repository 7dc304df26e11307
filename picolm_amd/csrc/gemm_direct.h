// The tile kernel whose tiles go from global memory straight into LDS, and its launcher: a
// template, so every file that names a variant compiles that variant.
#pragma once
#include "gemm_mfma.h"

// =============================================================================================
// tiled, with tiles loaded straight into LDS
// =============================================================================================
// The same block tiles and MFMA layout as the register-staged kernel of gemm_tiled.hip, but global
// memory is read by global_load_lds_dwordx4: a wave's 64 lanes bring 16 bytes each to 1 KB of LDS, with
// no staging registers and no LDS store instructions.  That leaves room for NS stages of BK
// columns, NS-1 of them in flight while one is multiplied, so that memory latency of several
// steps is covered by a single wave per SIMD.  The XOR swizzle is applied on the global side:
// the lane that fills LDS position p of a row fetches the chunk that belongs there.
//
// The loads are inline assembly so that the wait for "all but the newest steps" (s_waitcnt
// vmcnt(n)) stays as written: the compiler, when it knows of such loads, waits for all of them
// before any LDS read.  M0 carries the LDS address of a wave's 1 KB; nothing else here uses M0.
template <int BK>
__device__ __forceinline__ int swizzled_chunk(int row, int chunk) {
    return BK == 32 ? chunk ^ ((row >> 2) & 3) : chunk ^ ((row >> 1) & 7);
}
// The value that the lane named by a permutation of each four lanes holds (DPP quad_perm:
// 0xB1 the lane beside, 0x4E the lane two further on).
template <int QUAD_PERM>
__device__ __forceinline__ float swap_lanes(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), QUAD_PERM, 0xf, 0xf, true));
}
__device__ __forceinline__ void store_pair(float* p, float a, float b) { *(float2*)p = make_float2(a, b); }
__device__ __forceinline__ void store_pair(bf16_t* p, bf16_t a, bf16_t b) { *(unsigned*)p = (unsigned)a | ((unsigned)b << 16); }

// STREAM_SPREAD: the weights' loads that are spread between the MFMAs are non-temporal (a launch
// with one row of tiles, where every weight is read once).  A choice at compile time: made at run
// time at each of those loads it costs the long prompts' products 1.6 %.
template <int TN, int TM, int WN, int WM, int BK, int NS, int EPI, typename TC, bool STREAM_SPREAD = false>
__global__ __launch_bounds__(64 * WN * WM) void gemm_direct_kernel(const bf16_t* __restrict__ A,
                                                                   const bf16_t* __restrict__ W,
                                                                   TC* __restrict__ C, int M, int N, int K,
                                                                   int64_t lda, int64_t ldw, int64_t ldc,
                                                                   int tiles_m, int tiles_n, int64_t c_split_stride,
                                                                   NormLink link) {
    // the rows of the tile that a split norm keeps factors for: the sums' own 16 or 64 in a decode
    // step (one row of tiles), else all of the tile's
    __shared__ float link_scratch[64 * WN * WM], link_scale[32 * TM * WM > 64 ? 32 * TM * WM : 64];
    __shared__ float next_sums[EPI == 1 ? WN * 32 * TM * WM : 1];
    // K here is the length of one split: workgroup row y of the grid takes columns y*K .. of A
    // and W and writes its sums to C + y * c_split_stride
    A += (int64_t)blockIdx.y * K;
    W += (int64_t)blockIdx.y * K;
    C += (int64_t)blockIdx.y * c_split_stride;
    constexpr int NW = WN * WM;
    constexpr int BN = 32 * TN * WN, BM = 32 * TM * WM;
    constexpr int CH = BK / 8;                 // 16-byte chunks in a row of a stage
    constexpr int RG = 64 / CH;                // rows that one wave-wide load fills
    constexpr int STAGE = (BN + BM) * BK;      // bf16 elements
    constexpr int W_LOADS = BN / RG / NW, A_LOADS = BM / RG / NW;     // per wave and step
    static_assert((BN / RG) % NW == 0 && (BM / RG) % NW == 0, "tile does not split over the waves");
    extern __shared__ __attribute__((aligned(1024))) bf16_t lds[];
    int tile;
    {
        const int nb = gridDim.x, per = nb / 8, rem = nb % 8;
        const int xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
        tile = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
    }
    const int band = 8;
    const int per_band = band * tiles_m;
    const int b = tile / per_band, in_b = tile % per_band;
    const int band_w = min(band, tiles_n - b * band);
    const int tn = b * band + in_b % band_w, tm = in_b / band_w;
    const int n0 = tn * BN, m0 = tm * BM;
    const int link_rows = link.rows <= 64 ? link.rows : BM;
    const float link_mine = row_scale_begin<64 * WN * WM>(link, M, m0, link_rows);

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wn = (wave % WN) * (32 * TN), wm = (wave / WN) * (32 * TM);
    const int l32 = lane % 32, kq = lane / 32;

    // load j of a wave fills rows (j * NW + wave) * RG .. + RG - 1 of the W (then the A) tile
    const int lrow = lane / CH, lpos = lane % CH;
    unsigned w_off[W_LOADS], a_off[A_LOADS];
#pragma unroll
    for (int j = 0; j < W_LOADS; ++j) {
        const int row = (j * NW + wave) * RG + lrow;
        const int r = min(n0 + row, N - 1) - n0;
        w_off[j] = (unsigned)((r * ldw + swizzled_chunk<BK>(row, lpos) * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
        const int row = (j * NW + wave) * RG + lrow;
        const int r = min(m0 + row, M - 1) - m0;
        a_off[j] = (unsigned)((r * lda + swizzled_chunk<BK>(row, lpos) * 8) * 2);
    }
    const bf16_t* w_tile = W + (int64_t)n0 * ldw;
    const bf16_t* a_tile = A + (int64_t)m0 * lda;
    const unsigned lds_wave = __builtin_amdgcn_readfirstlane(
        (unsigned)(size_t)(__attribute__((address_space(3))) bf16_t*)lds + wave * (RG * BK * 2));
    // With one row of tiles every weight is read once, from memory: then workgroups start at
    // different places of K and wrap around.  If all of them walked K in step, all rows would be
    // read at the same column at the same time, and rows lie a power of two apart, so that few
    // memory channels would take all the traffic.  With several rows of tiles the tiles that share
    // a slice must stay in step, so that one of them finds it in L2.
    const int n_steps = K / BK;
    // with one row of tiles every weight is read once: past the caches
    const bool stream_w = tiles_m == 1;
    const int first_step = tiles_m == 1 ? (int)(((unsigned)tile * 5u + blockIdx.y * 3u) % (unsigned)n_steps) : 0;
    auto issue = [&](int stage, int step) {
        const unsigned to = lds_wave + stage * (STAGE * 2);
        step += first_step;
        if (step >= n_steps) step -= n_steps;
        const void* wsrc = same_in_every_lane(w_tile + step * BK);
        const void* asrc = same_in_every_lane(a_tile + step * BK);
        if (stream_w) {
#pragma unroll
            for (int j = 0; j < W_LOADS; ++j) stream_16_bytes_to_lds(w_off[j], wsrc, to + j * (NW * RG * BK * 2));
        } else {
#pragma unroll
            for (int j = 0; j < W_LOADS; ++j) load_16_bytes_to_lds(w_off[j], wsrc, to + j * (NW * RG * BK * 2));
        }
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) load_16_bytes_to_lds(a_off[j], asrc, to + (BN * BK * 2) + j * (NW * RG * BK * 2));
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // Fragments of k-slice g+1 are read from LDS while the MFMAs of slice g run; the wait, the
    // barrier and the next loads of a step sit in the middle of the last slice of the step before.
    constexpr int KS = BK / 16;
    constexpr bool SPREAD = TN * TM >= 4;      // the prefill's tiles (measured: 2 to 5 % for 256 x 256, nothing for the decode batches' tiles)
    static_assert(KS % 2 == 0, "fragment sets alternate by slice");
    bf16x8 wf[2][TN], af[2][TM];
    auto read_frags = [&](int stage, int ks, bf16x8 (&w)[TN], bf16x8 (&a)[TM]) {
        const bf16_t* Ws = lds + stage * STAGE;
        const bf16_t* As = Ws + BN * BK;
        const int chunk = ks * 2 + kq;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            const int row = wn + 32 * i + l32;
            w[i] = *(const bf16x8*)(Ws + row * BK + swizzled_chunk<BK>(row, chunk) * 8);
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int row = wm + 32 * j + l32;
            a[j] = *(const bf16x8*)(As + row * BK + swizzled_chunk<BK>(row, chunk) * 8);
        }
    };
    auto multiply = [&](const bf16x8 (&w)[TN], const bf16x8 (&a)[TM], int i_lo, int i_hi) {
#pragma unroll
        for (int i = i_lo; i < i_hi; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], w[i], acc[i][j], 0, 0, 0);
    };
    // K is a whole number of steps (the host sees to that).  Steps past the end load the last
    // step again into a stage nobody reads, so that the count of loads in flight stays the same.
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue(s, min(s, n_steps - 1));
    // begin step j: its loads have landed for every wave, the stage of step j-1 is read out and
    // takes the loads of step j+NS-1
    wait_for_loads<(W_LOADS + A_LOADS) * (NS - 2)>();
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    issue(NS - 1, min(NS - 1, n_steps - 1));
    read_frags(0, 0, wf[0], af[0]);
    int stage = 0;
    for (int it = 0; it < n_steps; ++it) {
        const int next_stage = stage + 1 == NS ? 0 : stage + 1;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + 1 < KS) {
                read_frags(stage, ks + 1, wf[(ks + 1) & 1], af[(ks + 1) & 1]);
                multiply(wf[ks & 1], af[ks & 1], 0, TN);
#pragma unroll
                for (int r = 0; r < TN + TM; ++r) {      // the reads early, one after each MFMA
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            } else if (SPREAD) {
                // The last slice begins with the wait and the barrier; the next loads follow one
                // by one between its MFMAs, each pinned where it is written: a burst of loads
                // holds up the MFMAs behind it while the memory pipeline takes them in.
                __builtin_amdgcn_sched_barrier(0);
                wait_for_loads<(W_LOADS + A_LOADS) * (NS - 2)>();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                const unsigned to = lds_wave + stage * (STAGE * 2);
                int step = min(it + NS, n_steps - 1) + first_step;
                if (step >= n_steps) step -= n_steps;
                const void* wsrc = same_in_every_lane(w_tile + step * BK);
                const void* asrc = same_in_every_lane(a_tile + step * BK);
                read_frags(next_stage, 0, wf[0], af[0]);       // past the last step: a stage of repeats
                __builtin_amdgcn_sched_barrier(0);
                constexpr int NL = W_LOADS + A_LOADS, NM = TN * TM, PER = (NL + NM - 1) / NM;
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int i = m / TM, j = m % TM;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][j], wf[ks & 1][i], acc[i][j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int q = 0; q < PER; ++q) {
                        const int l = m * PER + q;
                        if (l < W_LOADS) {
                            if constexpr (STREAM_SPREAD) stream_16_bytes_to_lds(w_off[l], wsrc, to + l * (NW * RG * BK * 2));
                            else load_16_bytes_to_lds(w_off[l], wsrc, to + l * (NW * RG * BK * 2));
                        } else if (l < NL) load_16_bytes_to_lds(a_off[l - W_LOADS], asrc, to + (BN * BK * 2) + (l - W_LOADS) * (NW * RG * BK * 2));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                multiply(wf[ks & 1], af[ks & 1], 0, TN / 2);
                __builtin_amdgcn_sched_barrier(0);
                wait_for_loads<(W_LOADS + A_LOADS) * (NS - 2)>();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                issue(stage, min(it + NS, n_steps - 1));
                read_frags(next_stage, 0, wf[0], af[0]);       // past the last step: a stage of repeats
                multiply(wf[ks & 1], af[ks & 1], TN / 2, TN);
#pragma unroll
                for (int r = 0; r < TN + TM; ++r) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        stage = next_stage;
    }
    wait_for_loads<0>();
    row_scale_finish<64 * WN * WM>(link, link_mine, link_rows, link_scratch, link_scale);
    // A product that adds into the residual rows can prepare the norm that follows (NormLink):
    // next_h = bf16(x * w) beside the new rows, and the tile's share of every row's sum of x^2.
    const bool prepares = EPI == 1 && link.next_w != nullptr;
    // The tile goes out in one of two ways: a tile that lies wholly inside C (most do) without a
    // test per element, a tile on the edge with them.  FULL is a type that says which.
    auto write_tile = [&](auto FULL) __attribute__((always_inline)) {
        constexpr bool full = decltype(FULL)::value;
        // element (i, j, e) of a lane is row r0 + 32j + 8(e/4) + e%4, column c0 + 32i of the tile
        const int r0 = wm + 4 * kq, c0 = wn + l32;
        TC* corner = C + (int64_t)m0 * ldc + (EPI == 2 ? n0 / 2 : n0);       // (n0 is even)
        bf16_t* hcorner = prepares ? link.next_h + (int64_t)m0 * ldc + n0 : nullptr;
        const unsigned ld = (unsigned)ldc;       // offsets within a tile fit 32 bits (the host sees to that)
        float next_w[TN];
#pragma unroll
        for (int i = 0; i < TN; ++i) next_w[i] = prepares && (full || n0 + c0 + 32 * i < N) ? link.next_w[n0 + c0 + 32 * i] : 0.f;
        if constexpr (EPI == 2) {
            // Two lanes side by side hold a gate column and its up column, 16 rows each.  They
            // swap half (DPP, no LDS): then the even lane has gate and up of its first eight rows
            // and the odd lane of its last eight, so that each value of the output is computed
            // once.  A second swap with the lane two further on, which holds the next output
            // column, leaves every lane two adjacent columns of four rows: four bytes a store.
            const int odd = l32 & 1, upper = (l32 >> 1) & 1;
            const int r0 = wm + 4 * kq + 16 * odd + 8 * upper;         // first of this lane's four rows in a block of 32
            const int oc = (wn >> 1) + ((l32 >> 2) << 1);              // lower of its two output columns, less 16 i
            TC* corner = C + (int64_t)m0 * ldc + n0 / 2;
            const unsigned ld = (unsigned)ldc;
            const bool paired = (ldc & 1) == 0 && ((uintptr_t)C & (2 * sizeof(TC) - 1)) == 0;     // (n0 / 2 is even)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int i = 0; i < TN; ++i) {
                    float o[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float lo = acc[i][j][k], hi = acc[i][j][k + 8];
                        const float recv = swap_lanes<0xB1>(odd ? lo : hi);      // with the lane beside
                        float g = odd ? recv : lo, u = odd ? hi : recv;
                        if (link.ssq) {
                            const int r = wm + 4 * kq + 32 * j + 16 * odd + 8 * (k / 4) + k % 4;
                            const float sc = (full || m0 + r < M) ? link_scale[r] : 0.f;
                            g *= sc;
                            u *= sc;
                        }
                        o[k] = silu_mul(g, u);
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float recv = swap_lanes<0x4E>(upper ? o[q] : o[q + 4]);   // with the lane two further
                        const float c_lo = upper ? recv : o[q], c_hi = upper ? o[q + 4] : recv;
                        const int r = r0 + 32 * j + q, c = oc + 16 * i;
                        if (!full && m0 + r >= M) continue;
                        TC* p = corner + (unsigned)r * ld + c;
                        const bool in_lo = full || n0 / 2 + c < N / 2, in_hi = full || n0 / 2 + c + 1 < N / 2;
                        if (paired && in_hi) {
                            store_pair(p, from_f32<TC>(c_lo), from_f32<TC>(c_hi));
                        } else {
                            if (in_lo) p[0] = from_f32<TC>(c_lo);
                            if (in_hi) p[1] = from_f32<TC>(c_hi);
                        }
                    }
                }
            return;
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            // what this product adds to: 32 rows' values are all asked for before the first is used
            float before[EPI == 1 ? TN : 1][16];
            if (EPI == 1) {
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int r = r0 + 32 * j + 8 * (e / 4) + e % 4, c = c0 + 32 * i;
                        const bool in = full || (m0 + r < M && n0 + c < N);
                        before[i][e] = in ? to_f32<TC>(corner[(unsigned)r * ld + c]) : 0.f;
                    }
            }
            float sq[16];               // this lane's share of 16 rows' sums of x^2
#pragma unroll
            for (int e = 0; e < 16; ++e) sq[e] = 0.f;
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                const int c = c0 + 32 * i;
                const bool c_in = full || n0 + c < N;
                unsigned hv[16];            // bf16(x * w) of this lane's 16 rows
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int r = r0 + 32 * j + 8 * (e / 4) + e % 4;
                    const bool r_in = full || m0 + r < M;
                    float v = acc[i][j][e];
                    if (link.ssq && r_in) v *= link_scale[r];
                    hv[e] = 0;
                    if (EPI == 2) {
                        const float up = __shfl_xor(v, 1, WAVE);
                        if (r_in && (l32 & 1) == 0 && (full || n0 + c + 1 < N))
                            corner[(unsigned)r * ld + c / 2] = from_f32<TC>(silu_mul(v, up));
                    } else if (r_in && c_in) {
                        const float x = EPI == 1 ? before[EPI == 1 ? i : 0][e] + v : v;
                        corner[(unsigned)r * ld + c] = from_f32<TC>(x);
                        if (prepares) {
                            hv[e] = f32_to_bf16_bits(x * next_w[i]);
                            sq[e] += x * x;
                        }
                    }
                }
                if (prepares) {
                    // Two lanes side by side hold two adjacent columns of 16 rows each: they swap
                    // half of them, so that each writes two columns of 8 rows, four bytes a store
                    // (N and the row stride are even: the host sees to that).
                    const int odd = l32 & 1;
#pragma unroll
                    for (int e = 0; e < 16; e += 2) {
                        const unsigned send = odd ? hv[e] : hv[e + 1];
                        const unsigned recv = (unsigned)__shfl_xor((int)send, 1, WAVE);
                        const int ee = e + odd;                 // the row this lane writes
                        const int r = r0 + 32 * j + 8 * (ee / 4) + ee % 4;
                        const unsigned lo = odd ? recv : hv[e], hi = odd ? hv[e + 1] : recv;
                        if (full || (m0 + r < M && n0 + c - odd + 1 < N))
                            *(unsigned*)(hcorner + (unsigned)r * ld + (c - odd)) = (lo & 0xffffu) | (hi << 16);
                    }
                }
            }
            if (prepares) {
                // The 16 rows' sums over the wave's columns, that is over the 32 lanes that hold
                // them.  Lanes that differ in one bit swap half of what they still hold and add,
                // four times: then a lane holds one row, the one its low four bits spell, summed
                // over 16 lanes; the lane 16 further on holds the rest of it.
#pragma unroll
                for (int half = 8; half >= 1; half /= 2) {
                    const int bit = 8 / half;               // 1, 2, 4, 8
                    const bool upper = (l32 & bit) != 0;    // this lane keeps the upper half
#pragma unroll
                    for (int k = 0; k < half; ++k) {
                        const float recv = __shfl_xor(upper ? sq[k] : sq[k + half], bit, WAVE);
                        sq[k] = (upper ? sq[k + half] : sq[k]) + recv;
                    }
                }
                const float t = sq[0] + __shfl_xor(sq[0], 16, WAVE);
                const int e = 8 * (l32 & 1) + 4 * ((l32 >> 1) & 1) + 2 * ((l32 >> 2) & 1) + ((l32 >> 3) & 1);
                if (l32 < 16) next_sums[(wave % WN) * BM + r0 + 32 * j + 8 * (e / 4) + e % 4] = t;
            }

        }
    };
    if (m0 + BM <= M && n0 + BN <= N) write_tile(std::true_type{});
    else write_tile(std::false_type{});
    if (EPI == 1 && prepares) {       // (uniform over the workgroup)
        // ... then over the waves side by side, in a fixed order
        __syncthreads();
        for (int r = tid; r < BM; r += 64 * WN * WM) {
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < WN; ++w) t += next_sums[w * BM + r];
            if (m0 + r < M) link.next_ssq[(size_t)tn * link.rows + m0 + r] = t;
        }
    }
}

template <int TN, int TM, int WN, int WM, int BK, int NS, bool MAY_STREAM_SPREAD = false>
static int launch_direct(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                         int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits = 1,
                         int64_t c_split_stride = 0, NormLink link = NormLink{}) {
    constexpr int BN = 32 * TN * WN, BM = 32 * TM * WM;
    // sums kept for 16 or 64 rows belong to a decode step, which has one row of tiles; otherwise
    // they are kept for every row
    PICOLM_REQUIRE((!link.ssq && !link.next_w) ||
                       (splits == 1 && M <= link.rows && (link.rows > 64 || ((link.rows == 16 || link.rows == 64) && M <= BM))),
                   "gemm_tiled: a split norm goes with an uncut product and sums for every row (%d rows, sums for %d)", M, link.rows);
    PICOLM_REQUIRE((int64_t)BM * ldc < (1ll << 29), "gemm_tiled: a row stride of %lld overflows the tile's 32-bit offsets", (long long)ldc);
    PICOLM_REQUIRE(!link.next_w || (N % 2 == 0 && ldc % 2 == 0 && ((uintptr_t)link.next_h & 3) == 0),
                   "gemm_tiled: preparing a norm writes pairs of columns: N and the row stride must be even");
    PICOLM_REQUIRE(!link.next_w || (epilogue == 1 && link.next_parts >= ceil_div(N, BN)),
                   "gemm_tiled: only the accumulating epilogue prepares a norm, one share of the sums per column of tiles");
    PICOLM_REQUIRE(splits >= 1 && K % (BK * splits) == 0,
                   "gemm_tiled: K = %d is no multiple of %d times %d splits, which this variant needs", K, BK, splits);
    PICOLM_REQUIRE((int64_t)BN * ldw < (1ll << 30) && (int64_t)BM * lda < (1ll << 30),
                   "gemm_tiled: row strides %lld / %lld overflow the tile's 32-bit offsets", (long long)lda, (long long)ldw);
    const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
    PICOLM_REQUIRE((int64_t)tiles_m * tiles_n < (1ll << 31), "gemm_tiled: too many tiles");
    dim3 grid(tiles_m * tiles_n, splits), block(64 * WN * WM);
    const size_t lds = (size_t)NS * (BN + BM) * BK * sizeof(bf16_t);
    static_assert((size_t)NS * (BN + BM) * BK * 2 <= 160 * 1024, "stages exceed the LDS");
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    const int k_len = K / splits;
#define TD_LAUNCH(EPI, TC)                                                                                 \
    {                                                                                                      \
        static size_t raised = 48 * 1024;                                                                  \
        if (lds > raised) {                                                                                \
            hipError_t e = hipFuncSetAttribute((const void*)gemm_direct_kernel<TN, TM, WN, WM, BK, NS, EPI, TC>, \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);      \
            if (e == hipSuccess && MAY_STREAM_SPREAD)                                                      \
                e = hipFuncSetAttribute((const void*)gemm_direct_kernel<TN, TM, WN, WM, BK, NS, EPI, TC, MAY_STREAM_SPREAD>, \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);             \
            PICOLM_REQUIRE(e == hipSuccess, "gemm_tiled: cannot raise the LDS limit: %s",                  \
                           hipGetErrorString(e));                                                          \
            raised = lds;                                                                                  \
        }                                                                                                  \
        if (MAY_STREAM_SPREAD && tiles_m == 1)                                                             \
            gemm_direct_kernel<TN, TM, WN, WM, BK, NS, EPI, TC, MAY_STREAM_SPREAD><<<grid, block, lds, stream>>>( \
                a, w, (TC*)C, M, N, k_len, lda, ldw, ldc, tiles_m, tiles_n, c_split_stride, link);         \
        else                                                                                               \
            gemm_direct_kernel<TN, TM, WN, WM, BK, NS, EPI, TC><<<grid, block, lds, stream>>>(             \
                a, w, (TC*)C, M, N, k_len, lda, ldw, ldc, tiles_m, tiles_n, c_split_stride, link);         \
    }
    if (epilogue == 0 && c_dt == PICOLM_F32) TD_LAUNCH(0, float)
    else if (epilogue == 0 && c_dt == PICOLM_BF16) TD_LAUNCH(0, bf16_t)
    else if (epilogue == 1 && c_dt == PICOLM_F32) TD_LAUNCH(1, float)
    else if (epilogue == 2 && c_dt == PICOLM_BF16) TD_LAUNCH(2, bf16_t)
    else if (epilogue == 2 && c_dt == PICOLM_F32) TD_LAUNCH(2, float)
    else PICOLM_REQUIRE(false, "gemm_tiled: unsupported epilogue %d with output dtype %d", epilogue, c_dt);
#undef TD_LAUNCH
    PICOLM_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

