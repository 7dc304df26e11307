// The tiled products (more than 16 rows), their cut along K and the entry points that choose
// between the kernels; see gemm_mfma.hip for the layout of operands.
#include "gemm_direct.h"

// =============================================================================================
// tiled
// =============================================================================================
// A block of WN x WM waves computes a (32*TN*WN) x (32*TM*WM) tile of C; a wave owns TN x TM MFMA
// tiles of 32 x 32.  Here the activation tile is the MFMA's first operand and the weight tile its
// second, so that an accumulator lane holds one column n and the 32 lanes of a half wave write
// 32 consecutive n of one row: stores are whole 128-byte runs.  K advances in steps of 64 through
// two LDS stages and two sets of staging registers: the loads of step it+2 are in flight while
// step it is multiplied and step it+1 is written to LDS; one barrier a step.  LDS rows are 64
// bf16 (128 bytes, half of the 64 banks); 16-byte chunk c of row r sits at c ^ ((r / 2) % 8), so
// that 16 consecutive rows of one chunk column touch every bank once.
#define TG_BK 64
#define TG_CHUNKS (TG_BK / 8)

__device__ __forceinline__ int tile_off(int row, int chunk) { return row * TG_BK + ((chunk ^ ((row >> 1) & 7)) << 3); }

template <int TN, int TM, int WN, int WM, int DEPTH, int EPI, typename TC>
__global__ __launch_bounds__(64 * WN * WM) void gemm_tiled_kernel(const bf16_t* __restrict__ A,
                                                                  const bf16_t* __restrict__ W,
                                                                  TC* __restrict__ C, int M, int N, int K,
                                                                  int64_t lda, int64_t ldw, int64_t ldc,
                                                                  int tiles_m, int tiles_n) {
    constexpr int THREADS = 64 * WN * WM;
    constexpr int BN = 32 * TN * WN, BM = 32 * TM * WM;
    constexpr int STAGE = (BN + BM) * TG_BK;
    constexpr int ROWS_PER_PASS = THREADS / TG_CHUNKS;
    constexpr int WP = BN / ROWS_PER_PASS, AP = BM / ROWS_PER_PASS;       // staging passes
    static_assert(BN % ROWS_PER_PASS == 0 && BM % ROWS_PER_PASS == 0, "tile does not split over the threads");
    extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
    // Workgroups are dealt to the 8 XCDs in turn and each XCD has an L2 of its own: workgroup b
    // takes the (b / 8)-th tile of XCD (b % 8)'s contiguous share, so that neighbours in tile
    // order meet in one L2.  Tile order walks down M inside a band of 8 tiles of N, so that a
    // band of weights stays in cache while activations stream.
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

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wn = (wave % WN) * (32 * TN), wm = (wave / WN) * (32 * TM);
    const int l32 = lane % 32, kq = lane / 32;

    // global -> register staging: a thread carries chunk `ld_chunk` of rows ld_row + ROWS_PER_PASS*i
    const int ld_chunk = tid % TG_CHUNKS, ld_row = tid / TG_CHUNKS;
    const bf16_t* wsrc[WP];
    const bf16_t* asrc[AP];
#pragma unroll
    for (int i = 0; i < WP; ++i) wsrc[i] = W + (int64_t)min(n0 + ld_row + ROWS_PER_PASS * i, N - 1) * ldw + ld_chunk * 8;
#pragma unroll
    for (int i = 0; i < AP; ++i) asrc[i] = A + (int64_t)min(m0 + ld_row + ROWS_PER_PASS * i, M - 1) * lda + ld_chunk * 8;
    bf16x8 wreg[DEPTH][WP], areg[DEPTH][AP];
    auto fetch = [&](bf16x8 (&wr)[WP], bf16x8 (&ar)[AP], int k0) {      // a whole step inside K
#pragma unroll
        for (int i = 0; i < WP; ++i) wr[i] = load_chunk(wsrc[i] + k0);
#pragma unroll
        for (int i = 0; i < AP; ++i) ar[i] = load_chunk(asrc[i] + k0);
    };
    auto fetch_any = [&](bf16x8 (&wr)[WP], bf16x8 (&ar)[AP], int k0) {  // chunks past K are zero
        const bool kvalid = k0 + ld_chunk * 8 < K;
#pragma unroll
        for (int i = 0; i < WP; ++i) wr[i] = kvalid ? load_chunk(wsrc[i] + k0) : zero_chunk();
#pragma unroll
        for (int i = 0; i < AP; ++i) ar[i] = kvalid ? load_chunk(asrc[i] + k0) : zero_chunk();
    };
    auto stash = [&](const bf16x8 (&wr)[WP], const bf16x8 (&ar)[AP], int stage) {
        bf16_t* Ws = lds + stage * STAGE;
        bf16_t* As = Ws + BN * TG_BK;
#pragma unroll
        for (int i = 0; i < WP; ++i) *(bf16x8*)(Ws + tile_off(ld_row + ROWS_PER_PASS * i, ld_chunk)) = wr[i];
#pragma unroll
        for (int i = 0; i < AP; ++i) *(bf16x8*)(As + tile_off(ld_row + ROWS_PER_PASS * i, ld_chunk)) = ar[i];
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    auto compute = [&](int stage) {
        const bf16_t* Ws = lds + stage * STAGE;
        const bf16_t* As = Ws + BN * TG_BK;
#pragma unroll
        for (int ks = 0; ks < TG_BK / 16; ++ks) {
            const int chunk = ks * 2 + kq;
            bf16x8 wf[TN], af[TM];
#pragma unroll
            for (int i = 0; i < TN; ++i) wf[i] = *(const bf16x8*)(Ws + tile_off(wn + 32 * i + l32, chunk));
#pragma unroll
            for (int j = 0; j < TM; ++j) af[j] = *(const bf16x8*)(As + tile_off(wm + 32 * j + l32, chunk));
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[j], wf[i], acc[i][j], 0, 0, 0);
        }
    };
    // Steps are numbered 0 .. n_iter-1; the last one may be partial.  The steady-state loop has
    // no branch between a load and its use (a branch there makes the compiler wait for the loads
    // at once) and scheduling barriers keep the loads where they are written.
    const int n_iter = (K + TG_BK - 1) / TG_BK;
    const int n_full = K / TG_BK;
    fetch_any(wreg[0], areg[0], 0);
    stash(wreg[0], areg[0], 0);
    int cur = 0, it = 0;
    if (DEPTH == 2) {
        if (n_iter > 1) fetch_any(wreg[0], areg[0], TG_BK);       // step 1, in flight
        __syncthreads();
        int held = 0;                                              // the register set with step it+1
        while (it + 3 < n_full) {                                   // steps it+2 and it+3 are whole
            fetch(wreg[DEPTH - 1], areg[DEPTH - 1], (it + 2) * TG_BK);
            __builtin_amdgcn_sched_barrier(0);
            compute(cur);
            __builtin_amdgcn_sched_barrier(0);
            stash(wreg[0], areg[0], cur ^ 1);
            __syncthreads();
            fetch(wreg[0], areg[0], (it + 3) * TG_BK);
            __builtin_amdgcn_sched_barrier(0);
            compute(cur ^ 1);
            __builtin_amdgcn_sched_barrier(0);
            stash(wreg[DEPTH - 1], areg[DEPTH - 1], cur);
            __syncthreads();
            it += 2;
        }
        while (it < n_iter) {                                       // the last steps, one at a time
            if (it + 2 < n_iter) {
                if (held == 0) fetch_any(wreg[DEPTH - 1], areg[DEPTH - 1], (it + 2) * TG_BK);
                else fetch_any(wreg[0], areg[0], (it + 2) * TG_BK);
            }
            compute(cur);
            if (it + 1 < n_iter) {
                if (held == 0) stash(wreg[0], areg[0], cur ^ 1);
                else stash(wreg[DEPTH - 1], areg[DEPTH - 1], cur ^ 1);
                __syncthreads();
                cur ^= 1;
                held ^= 1;
            }
            ++it;
        }
    } else {
        __syncthreads();
        while (it + 1 < n_full) {                                   // step it+1 is whole
            fetch(wreg[0], areg[0], (it + 1) * TG_BK);
            __builtin_amdgcn_sched_barrier(0);
            compute(cur);
            __builtin_amdgcn_sched_barrier(0);
            stash(wreg[0], areg[0], cur ^ 1);
            __syncthreads();
            cur ^= 1;
            ++it;
        }
        while (it < n_iter) {
            if (it + 1 < n_iter) fetch_any(wreg[0], areg[0], (it + 1) * TG_BK);
            compute(cur);
            if (it + 1 < n_iter) {
                stash(wreg[0], areg[0], cur ^ 1);
                __syncthreads();
                cur ^= 1;
            }
            ++it;
        }
    }
    // accumulator element e of tile (i, j): m = wm + 32j + 8*(e/4) + 4*kq + e%4, n = wn + 32i + l32
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        const int n = n0 + wn + 32 * i + l32;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm + 32 * j + 8 * (e / 4) + 4 * kq + e % 4;
                const float v = acc[i][j][e];
                if (EPI == 2) {
                    // gate at even n, up at odd n: the odd lane hands its value to the even one
                    const float up = __shfl_xor(v, 1, WAVE);
                    if (m < M && (l32 & 1) == 0 && n + 1 < N) C[(int64_t)m * ldc + n / 2] = from_f32<TC>(silu_mul(v, up));
                } else if (m < M && n < N) {
                    TC* p = C + (int64_t)m * ldc + n;
                    *p = from_f32<TC>(EPI == 1 ? to_f32<TC>(*p) + v : v);
                }
            }
        }
    }
}

template <int TN, int TM, int WN, int WM, int DEPTH>
static int launch_tiled(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                        int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream) {
    constexpr int BN = 32 * TN * WN, BM = 32 * TM * WM;
    const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
    PICOLM_REQUIRE((int64_t)tiles_m * tiles_n < (1ll << 31), "gemm_tiled: too many tiles");
    dim3 grid(tiles_m * tiles_n), block(64 * WN * WM);
    const size_t lds = 2 * (size_t)(BN + BM) * TG_BK * sizeof(bf16_t);
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
#define TG_LAUNCH(EPI, TC)                                                                                 \
    {                                                                                                      \
        static size_t raised = 48 * 1024;                                                                  \
        if (lds > raised) {                                                                                \
            hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<TN, TM, WN, WM, DEPTH, EPI, TC>,    \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);      \
            PICOLM_REQUIRE(e == hipSuccess, "gemm_tiled: cannot raise the LDS limit: %s",                  \
                           hipGetErrorString(e));                                                          \
            raised = lds;                                                                                  \
        }                                                                                                  \
        gemm_tiled_kernel<TN, TM, WN, WM, DEPTH, EPI, TC><<<grid, block, lds, stream>>>(a, w, (TC*)C, M, N, K, lda, \
                                                                                ldw, ldc, tiles_m, tiles_n); \
    }
    if (epilogue == 0 && c_dt == PICOLM_F32) TG_LAUNCH(0, float)
    else if (epilogue == 0 && c_dt == PICOLM_BF16) TG_LAUNCH(0, bf16_t)
    else if (epilogue == 1 && c_dt == PICOLM_F32) TG_LAUNCH(1, float)
    else if (epilogue == 2 && c_dt == PICOLM_BF16) TG_LAUNCH(2, bf16_t)
    else if (epilogue == 2 && c_dt == PICOLM_F32) TG_LAUNCH(2, float)
    else PICOLM_REQUIRE(false, "gemm_tiled: unsupported epilogue %d with output dtype %d", epilogue, c_dt);
#undef TG_LAUNCH
    PICOLM_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

// ---- split K ---------------------------------------------------------------------------------
// A product with few output tiles is cut along K so that every CU has a workgroup: split z
// writes its partial sums to ws[z][M][N]; the kernel below adds the splits in order (the same
// order every time) and applies the epilogue.
// With a split norm (NormLink) N is a multiple of 1024, so that the 1024 values of a workgroup lie
// in one row: as the consumer it multiplies the sums by the row's factor; as the producer (epilogue
// 1) it leaves bf16(x * w) and one partial sum of x^2 per workgroup.
template <int EPI, typename TC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, TC* __restrict__ C, int M, int N,
                                                            int64_t ldc, int splits, NormLink link) {
    __shared__ float wave_sq[4];
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;      // four floats of a row
    const bool inside = i < (int64_t)M * N;      // (always, with a split norm)
    const int m = inside ? (int)(i / N) : 0, n = inside ? (int)(i % N) : 0;      // N is a multiple of 4 (the host sees to that)
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (inside)
        for (int z0 = 0; z0 < splits; z0 += 8) {      // eight parts asked for at a time, added in order
            f32x4 part[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) part[e] = *(const f32x4*)(ws + (int64_t)min(z0 + e, splits - 1) * M * N + i);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (z0 + e < splits) sum += part[e];
        }
    if (link.ssq) {
        float total = 0.f;      // (eight loads asked for at a time, as in row_scale_begin)
        for (int p0 = 0; p0 < link.n_parts; p0 += 8) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = link.ssq[(size_t)min(p0 + e, link.n_parts - 1) * link.rows + m];
#pragma unroll
            for (int e = 0; e < 8; ++e) total += p0 + e < link.n_parts ? v[e] : 0.f;
        }
        sum *= 1.0f / sqrtf(total * link.inv_len + link.eps);
    }
    float sq = 0.f;
    if (inside) {
        if (EPI == 2) {
            TC* p = C + (int64_t)m * ldc + n / 2;
            p[0] = from_f32<TC>(silu_mul(sum[0], sum[1]));
            p[1] = from_f32<TC>(silu_mul(sum[2], sum[3]));
        } else {
            TC* p = C + (int64_t)m * ldc + n;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x = EPI == 1 ? to_f32<TC>(p[e]) + sum[e] : sum[e];
                p[e] = from_f32<TC>(x);
                if (EPI == 1 && link.next_w) {
                    link.next_h[(int64_t)m * ldc + n + e] = f32_to_bf16_bits(x * link.next_w[n + e]);
                    sq += x * x;
                }
            }
        }
    }
    if (EPI == 1 && link.next_w) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
        if (threadIdx.x % 64 == 0) wave_sq[threadIdx.x / 64] = sq;
        __syncthreads();
        if (threadIdx.x == 0)
            link.next_ssq[(size_t)(blockIdx.x % (N / 1024)) * link.rows + m] = wave_sq[0] + wave_sq[1] + wave_sq[2] + wave_sq[3];
    }
}

static int launch_splitk_reduce(const float* ws, void* C, int c_dt, int M, int N, int64_t ldc, int splits, int epilogue,
                                hipStream_t stream, NormLink link) {
    PICOLM_REQUIRE((!link.ssq && !link.next_w) || (N % 1024 == 0 && M <= link.rows),
                   "gemm_splitk: a split norm needs N (%d) in multiples of 1024 and up to %d rows", N, link.rows);
    PICOLM_REQUIRE(!link.next_w || (epilogue == 1 && link.next_parts >= N / 1024),
                   "gemm_splitk: only the accumulating epilogue prepares a norm");
    const int64_t quads = (int64_t)M * N / 4;
    dim3 grid((unsigned)ceil_div64(quads, 256)), block(256);
    if (epilogue == 0 && c_dt == PICOLM_F32) splitk_reduce_kernel<0, float><<<grid, block, 0, stream>>>(ws, (float*)C, M, N, ldc, splits, link);
    else if (epilogue == 0 && c_dt == PICOLM_BF16) splitk_reduce_kernel<0, bf16_t><<<grid, block, 0, stream>>>(ws, (bf16_t*)C, M, N, ldc, splits, link);
    else if (epilogue == 1 && c_dt == PICOLM_F32) splitk_reduce_kernel<1, float><<<grid, block, 0, stream>>>(ws, (float*)C, M, N, ldc, splits, link);
    else if (epilogue == 2 && c_dt == PICOLM_BF16) splitk_reduce_kernel<2, bf16_t><<<grid, block, 0, stream>>>(ws, (bf16_t*)C, M, N, ldc, splits, link);
    else if (epilogue == 2 && c_dt == PICOLM_F32) splitk_reduce_kernel<2, float><<<grid, block, 0, stream>>>(ws, (float*)C, M, N, ldc, splits, link);
    else PICOLM_REQUIRE(false, "gemm_splitk: unsupported epilogue %d with output dtype %d", epilogue, c_dt);
    PICOLM_LAUNCH_CHECK("gemm_splitk_reduce");
    return 0;
}

// variant 0 picks by shape.  Tiles loaded straight into LDS (K a multiple of 64):
//   9: 256x256, 8 waves, two stages of 64 columns;  10: 256(n)x128(m), 8 waves, three stages;
//   11: 128x128, 4 waves, four stages;  14: 192(n)x256(m), 15: 320(n)x256(m), 8 waves, two stages;
//   12: 128(n)x64(m), 4 waves, three stages;  13: 128(n)x32(m), 4 waves, four stages: for decode
//   batches of up to 64 or 32 rows, where the weights stream once and K may be split.
// Tiles staged through registers (any K that is a multiple of 8):
//   1: 128x128 (4 waves), 4: 256x256 (8 waves).
// The tile variant for a product by its shape.  Every variant moves about the same bytes a second
// from L2 into LDS, so the largest tile wins once its workgroups fill most of the 256 CUs.
// n_first > 0: the first n_first columns of 256x256 tiles go to variant 9 and the rest to variant
// 10: a last round that fills half of the CUs or less costs nearly a whole round, and the 256x128
// tile gives those columns twice the workgroups.
static int tiled_plan_256(int M, int N, int K, int& n_first) {
    n_first = 0;
    const int tiles_m = ceil_div(M, 256), tiles_n = ceil_div(N, 256);
    const int64_t t256 = (int64_t)tiles_m * tiles_n;
    const int64_t t128m = (int64_t)ceil_div(M, 128) * tiles_n;
    if (K % 64 != 0) return t256 >= 512 ? 4 : 1;
    const int64_t whole = t256 / 256 * 256, left = t256 - whole;
    const int first = (int)(whole / tiles_m);
    const int64_t rest = (int64_t)(tiles_n - first) * ceil_div(M, 128);
    if (whole > 0 && left > 0 && left <= 160 && first > 0 && rest <= 288) {
        n_first = first;
        return 9;
    }
    return t256 >= 144 ? 9 : t128m >= 144 ? 10 : 11;
}
// Where N is a whole number of 192 columns (the qkv product of 32 + 8 + 8 heads of 128), tiles of
// 192 columns by 256 rows (variant 14) may fill the CUs' rounds better than 256 x 256: 2,048 rows of
// 6,144 columns are 192 tiles of the one kind, three quarters of a round, and exactly 256 of the
// other.  Likewise 320 columns (variant 15) for 10,240 (64 + 8 + 8 heads): 320 tiles or 256.  The plans are compared by their rounds weighted with the tile's size (a 256 x 128 tile
// does a little more than half the work of a 256 x 256 tile's time, a 192-column tile three
// quarters and a little); measured at 1,024 to 16,384 rows of the qkv shape, the rule takes the
// faster plan everywhere (15 % at 1,536 rows, 6 % at 2,048, 5 % at 3,072 and 6,144).
static int tiled_plan(int M, int N, int K, int epilogue, int& n_first) {
    const int variant = tiled_plan_256(M, N, K, n_first);
    if (K % 64 != 0 || variant == 11) return variant;
    const int tiles_m = ceil_div(M, 256);
    const int64_t t256 = (int64_t)tiles_m * ceil_div(N, 256);
    double cost;
    if (n_first > 0)
        cost = (double)(t256 / 256) + 0.55 * (double)ceil_div64((int64_t)(ceil_div(N, 256) - n_first) * ceil_div(M, 128), 256);
    else if (variant == 9)
        cost = (double)ceil_div64(t256, 256);
    else
        cost = 0.55 * (double)ceil_div64((int64_t)ceil_div(M, 128) * ceil_div(N, 256), 256);
    // tiles of 192 or 320 columns (variants 14, 15) where the columns are a whole number of them:
    // their rounds times the width's share of 256, a little more for the narrow tile and a little
    // less for the wide one, which moves fewer bytes per flop (1.35 against 1.22 PFLOP/s at 8,192
    // rows of 10,240 columns).  The wide tile's sums fill the registers: not with the epilogue that
    // adds to what is there, which needs room of its own.
    int best = variant;
    for (int width : {192, 320}) {
        if (N % width != 0 || (width == 320 && epilogue == 1)) continue;
        const int64_t t = (int64_t)tiles_m * (N / width);
        const double c = (width == 192 ? 1.03 : 0.93) * width / 256.0 * (double)ceil_div64(t, 256);
        if (t >= 144 && c <= cost) {
            cost = c;
            best = width == 192 ? 14 : 15;
        }
    }
    if (best != variant) n_first = 0;
    return best;
}

// A short prompt's product with a narrow output has tiles for half of the CUs or fewer (512 rows
// and 4096 columns: 128 tiles of 128x128).  Given room for the parts' sums it is cut along K like
// a wide decode batch's, into 2, 4 or 8 (no more workgroups than CUs: 80 tiles of 256 x 5,120 x
// 13,824 cut in two take 78.5 us, in four 85.9), and the adding kernel applies the epilogue.  The cut depends
// on the shape and the room alone, not on whether a norm is split around the product: the shares
// of a norm's sums (N / 1024 of the adding kernel) must be known before the call.
static int tiled_splits(int M, int N, int K, int variant, int64_t ws_floats) {
    if (variant < 9 || variant > 11 || N % 1024 != 0) return 1;
    const int bn = variant == 11 ? 128 : 256, bm = variant == 9 ? 256 : 128;
    const int64_t tiles = (int64_t)ceil_div(M, bm) * ceil_div(N, bn);
    if (tiles > 128) return 1;
    int s = 8;
    while (s > 1 && (tiles * s > n_compute_units() || K % (64 * s) != 0 || (int64_t)s * M * N > ws_floats)) s /= 2;
    return s;
}

// The variant, the cut along K and the two-launch plan for a shape.  Where the 128x128 tiles are
// too many to cut but the 256x128 ones are few and K is long (a prompt of 768 tokens into the
// model's width from the feed-forward's), the larger tile cut in two is the faster (measured
// 103 against 114 us at 768 x 4096 x 14336 and 135 against 140 at 1024 rows; with K = 4096 the
// smaller tile uncut wins, and with K = 8192 too: 76 against 82 us at 2048 x 2048 x 8192).
static void tiled_choice(int M, int N, int K, int epilogue, int64_t ws_floats, int& variant, int& splits, int& n_first) {
    variant = tiled_plan(M, N, K, epilogue, n_first);
    splits = 1;
    if (n_first > 0) return;
    splits = tiled_splits(M, N, K, variant, ws_floats);
    if (splits == 1 && variant == 11 && K > 8192) {
        const int s10 = tiled_splits(M, N, K, 10, ws_floats);
        if (s10 > 1) {
            variant = 10;
            splits = s10;
        }
    }
}

// Shares of a row's sum of squares that the tiled product of this shape leaves when it prepares a
// norm (one per column of tiles, or per 1024 columns if the product is cut along K, which it is
// when a workspace of ws_floats floats allows it), or 0 if its kernel cannot take part in a split norm.
extern "C" int picolm_gemm_tiled_norm_parts(int M, int N, int K, int64_t ws_floats) {
    int variant, splits, n_first;
    tiled_choice(M, N, K, 1, ws_floats, variant, splits, n_first);       // the product that prepares a norm adds to the rows
    if (splits > 1) return N % 1024 ? 0 : N / 1024;      // the kernel that adds the parts takes 1024 columns a workgroup
    if (N % 2) return 0;                                 // the tile kernels write the next rows in pairs of columns
    return variant == 9 || variant == 10 ? ceil_div(N, 256) : variant == 11 ? ceil_div(N, 128) : variant == 14 ? ceil_div(N, 192) : variant == 15 ? ceil_div(N, 320) : 0;
}

static int launch_splitk_reduce(const float* ws, void* C, int c_dt, int M, int N, int64_t ldc, int splits, int epilogue,
                                hipStream_t stream, NormLink link);
static int gemm_tiled_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                             int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link,
                             float* ws = nullptr, int64_t ws_floats = 0);

extern "C" int picolm_gemm_tiled(const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                 int64_t lda, int64_t ldw, int64_t ldc, int epilogue, int variant,
                                 hipStream_t stream) {
    if (check_mfma_operands("gemm_tiled", A, W, M, N, K, lda, ldw, ldc, epilogue, c_dt)) return -1;
    if (M == 0) return 0;
    return gemm_tiled_linked(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, variant, stream, NormLink{});
}

static int gemm_tiled_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                             int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link,
                             float* ws, int64_t ws_floats) {
    if (variant == 0) {
        int n_first, splits;
        tiled_choice(M, N, K, epilogue, ws != nullptr ? ws_floats : 0, variant, splits, n_first);
        if (splits > 1) {
            PICOLM_REQUIRE(((uintptr_t)ws & 15) == 0, "gemm_tiled: the workspace of a cut product must be 16-byte aligned");
            const int rc = picolm_gemm_direct_prefill_(variant, A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits,
                                                       (int64_t)M * N, NormLink{});
            if (rc) return rc;
            return launch_splitk_reduce(ws, C, c_dt, M, N, ldc, splits, epilogue, stream, link);
        }
        if (n_first > 0) {
            const int N1 = n_first * 256;
            const size_t c_item = c_dt == PICOLM_F32 ? 4 : 2;
            const int rc = gemm_tiled_linked(A, W, C, c_dt, M, N1, K, lda, ldw, ldc, epilogue, 9, stream, link);
            if (rc) return rc;
            if (link.next_w) {          // the second launch goes on where the first one's columns end
                link.next_w += N1;
                link.next_h += N1;
                link.next_ssq += (size_t)n_first * link.rows;
                link.next_parts -= n_first;
            }
            return gemm_tiled_linked(A, (const bf16_t*)W + (int64_t)N1 * ldw,
                                     (char*)C + c_item * (epilogue == 2 ? N1 / 2 : N1), c_dt, M, N - N1, K, lda, ldw,
                                     ldc, epilogue, 10, stream, link);
        }
    }
    if (link.ssq || link.next_w)
        PICOLM_REQUIRE((variant >= 9 && variant <= 11) || variant == 14 || variant == 15, "gemm_tiled: tile variant %d takes no part in a split norm", variant);
    switch (variant) {
        case 1: return launch_tiled<2, 2, 2, 2, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 4: return launch_tiled<2, 4, 4, 2, 1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 9: return picolm_gemm_direct_prefill_(9, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 10: return picolm_gemm_direct_prefill_(10, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 11: return picolm_gemm_direct_prefill_(11, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 14: return picolm_gemm_direct_prefill_(14, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 15: return picolm_gemm_direct_prefill_(15, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 12: return launch_direct<1, 2, 4, 1, 64, 3>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 13: return launch_direct<1, 1, 4, 1, 64, 4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
    }
    PICOLM_REQUIRE(false, "gemm_tiled: unknown variant %d", variant);
}

// The tiled product cut into `splits` along K (variants 9 and up only); ws holds
// splits * M * N floats.  N must be a multiple of 4.
extern "C" int picolm_gemm_tiled_splitk(const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                        int64_t lda, int64_t ldw, int64_t ldc, int epilogue, int variant,
                                        int splits, float* ws, hipStream_t stream) {
    if (check_mfma_operands("gemm_splitk", A, W, M, N, K, lda, ldw, ldc, epilogue, c_dt)) return -1;
    PICOLM_REQUIRE(splits >= 1 && splits <= 64, "gemm_splitk: %d splits", splits);
    if (splits == 1) return picolm_gemm_tiled(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, variant, stream);
    PICOLM_REQUIRE(ws != nullptr && ((uintptr_t)ws & 15) == 0, "gemm_splitk: needs a 16-byte aligned workspace");
    PICOLM_REQUIRE(N % 4 == 0, "gemm_splitk: N = %d is no multiple of 4", N);
    if (M == 0) return 0;
    const int64_t stride = (int64_t)M * N;
    int rc;
    switch (variant) {
        case 9: rc = picolm_gemm_direct_prefill_(9, A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride, NormLink{}); break;
        case 10: rc = picolm_gemm_direct_prefill_(10, A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride, NormLink{}); break;
        case 11: rc = picolm_gemm_direct_prefill_(11, A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride, NormLink{}); break;
        case 12: rc = launch_direct<1, 2, 4, 1, 64, 3>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        case 13: rc = launch_direct<1, 1, 4, 1, 64, 4>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        default: PICOLM_REQUIRE(false, "gemm_splitk: variant %d cannot split K", variant);
    }
    if (rc) return rc;
    return launch_splitk_reduce(ws, C, c_dt, M, N, ldc, splits, epilogue, stream, NormLink{});
}

// The products of a decode step with a norm split between them (see NormLink).  Up to 16 rows:
// `variant` as in picolm_gemm_skinny (0 or 1) or, with tiled != 0, tile variant 12 or 13; rows = 16.
// More than 64 rows (a prefill step): tiled, rows = a multiple of 64 of at least M, the tile
// variant by shape, cut along K if ws is given and the shape has few tiles; either role, the
// shares of the sums as picolm_gemm_tiled_norm_parts says for the same ws_floats.
// 17 to 64 rows: tiled, variant 12 (13 up to 32 rows), rows = 64; with splits > 1 (ws as in picolm_gemm_tiled_splitk)
// the kernel that adds the parts takes either role and N must be a multiple of 1024; uncut, the
// tile kernel can only take a prepared norm's statistics.
// next_*: this product (epilogue 1) prepares the norm that follows: next_h[M][ldc] and
// next_ssq[next_parts][rows], one row of partial sums per workgroup (ceil(N/16) of the skinny
// kernel, N/1024 of the adding kernel).  ssq, n_parts, norm_len, eps: this product's input rows
// are the next_h of a product that prepared their norm.
extern "C" int picolm_gemm_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                  int64_t ldw, int64_t ldc, int epilogue, int tiled, int variant, int splits,
                                  float* ws, int64_t ws_floats, const float* next_w, void* next_h, float* next_ssq, int next_parts,
                                  const float* ssq, int n_parts, int norm_len, float eps, int rows,
                                  hipStream_t stream) {
    if (check_mfma_operands("gemm_linked", A, W, M, N, K, lda, ldw, ldc, epilogue, c_dt)) return -1;
    PICOLM_REQUIRE((rows == 16 || rows == 64 || (rows > 64 && rows % 64 == 0)) && M <= rows,
                   "gemm_linked: %d rows with sums kept for %d", M, rows);
    PICOLM_REQUIRE(!next_w || (next_h && next_ssq && next_parts > 0), "gemm_linked: an incomplete description of the next norm");
    PICOLM_REQUIRE(!ssq || (n_parts > 0 && norm_len > 0), "gemm_linked: an incomplete description of the norm's statistics");
    PICOLM_REQUIRE(splits >= 1 && splits <= 64, "gemm_linked: %d splits", splits);
    if (M == 0) return 0;
    NormLink link = {next_w, (bf16_t*)next_h, next_ssq, next_parts, ssq, n_parts, norm_len > 0 ? 1.0f / (float)norm_len : 0.f, eps, rows};
    if (rows > 64) {            // a prefill step: the tile variants by shape, sums for every row
        PICOLM_REQUIRE(tiled && splits == 1, "gemm_linked: more than 64 rows take the uncut tiled product");
        return gemm_tiled_linked(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, 0, stream, link, ws, ws_floats);
    }
    if (tiled && splits > 1) {
        PICOLM_REQUIRE((int64_t)splits * M * N <= ws_floats, "gemm_linked: %d splits of %d x %d exceed the workspace", splits, M, N);
        PICOLM_REQUIRE((variant == 12 || (variant == 13 && M <= 32)) && ws != nullptr && ((uintptr_t)ws & 15) == 0 && N % 4 == 0,
                       "gemm_linked: a cut product needs tile variant 12 (or 13 up to 32 rows), a workspace and N in multiples of 4");
        const int rc = variant == 12
            ? launch_direct<1, 2, 4, 1, 64, 3>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, (int64_t)M * N)
            : launch_direct<1, 1, 4, 1, 64, 4>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, (int64_t)M * N);
        if (rc) return rc;
        return launch_splitk_reduce(ws, C, c_dt, M, N, ldc, splits, epilogue, stream, link);
    }
    if (tiled) {
        switch (variant) {
            case 12: return launch_direct<1, 2, 4, 1, 64, 3>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
            case 13: return launch_direct<1, 1, 4, 1, 64, 4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        }
        PICOLM_REQUIRE(false, "gemm_linked: tile variant %d cannot take a norm's statistics", variant);
    }
    return picolm_gemm_skinny_linked_(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, variant, stream, link);
}
