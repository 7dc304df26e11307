// bf16 x bf16 -> float products on the matrix cores of gfx950: C[M,N] = A[M,K] * W[N,K]^T.
//
// The skinny kernel feeds the weight tile as the MFMA's first operand and the activation tile
// as its second, so an accumulator lane holds four consecutive output columns n of one row m
// and gate/up pairs of the row-interleaved gated layout meet in one lane.
//
//   skinny (M <= 64, the decode step): HBM-bound.  A wave streams 16*NT weight rows straight
//     from global memory into MFMA operand registers, 16 bytes a lane; the waves of a block
//     split K between them and reduce through LDS.  Every weight byte is read once.
//   tiled (M > 64, the prefill step; gemm_tiled.hip, gemm_direct.h): block tiles of 128x128 to 256x256 in LDS with an XOR swizzle
//     of 16-byte chunks, 32x32x16 MFMAs; here the activation tile is the first operand, so that
//     stores are whole 128-byte runs.  Tiles reach LDS straight from global memory
//     (global_load_lds) when K is a multiple of 64, else through staging registers.  These
//     kernels are bound by what L2 delivers to the CUs, not by the matrix cores.
//
// The order of the K summation inside an MFMA does not matter, so a lane's 8-element chunk
// may come from any K offset as long as both operands use the same offset.
#include "gemm_mfma.h"

// =============================================================================================
// skinny
// =============================================================================================
#define SK_KSTEP 128      // K elements one wave consumes per step: 4 MFMAs of 32

// The values a thread of a skinny product's workgroup finishes, one per pass of the epilogue's
// loop: value v = ((t*MT + u)*4 + r)*64 + l is row m = 16 u + l % 16, column n_base + 16 t +
// 4 (l / 16) + r (the gated epilogue takes r and r + 1 together).
template <int MT, int NT, int WAVES, int EPI>
struct SkinnyValues {
    static constexpr int PER_WAVE = NT * MT * 4 * 64;
    static constexpr int STEP = (EPI == 2) ? 2 : 1;
    static constexpr int PASSES = (PER_WAVE / STEP + WAVES * 64 - 1) / (WAVES * 64);
    // where pass p's value lies: false if this thread has none there
    __device__ static bool place(int pass, int M, int N, int n_base, int rows_per_wg, int& idx, int& m, int& n) {
        const int v = threadIdx.x + pass * (WAVES * 64);
        if (v >= PER_WAVE / STEP) return false;
        const int l = v % 64;
        const int r = EPI == 2 ? 2 * ((v / 64) % 2) : (v / 64) % 4;
        const int tu = EPI == 2 ? v / 128 : v / 256;
        const int u = tu % MT, t = tu / MT;
        idx = ((t * MT + u) * 4 + r) * 64 + l;
        n = n_base + t * 16 + 4 * (l / 16) + r;
        m = u * 16 + l % 16;
        return m < M && n < N && t * 16 + 4 * (l / 16) + r < rows_per_wg;
    }
    float before[PASSES], next_w[PASSES];      // (accumulating epilogue) what the sums are added to, the next norm's weight
};
// Asked for before the main loop, so that the epilogue does not wait a trip to memory for them.
template <int MT, int NT, int WAVES, int EPI, typename TC>
__device__ __forceinline__ SkinnyValues<MT, NT, WAVES, EPI> skinny_prefetch(const TC* __restrict__ C, int M, int N, int64_t ldc,
                                                                            const NormLink& link, int n_base, int rows_per_wg) {
    SkinnyValues<MT, NT, WAVES, EPI> pre;
#pragma unroll
    for (int pass = 0; pass < pre.PASSES; ++pass) {
        pre.before[pass] = pre.next_w[pass] = 0.f;
        int idx, m, n;
        if (EPI == 1 && pre.place(pass, M, N, n_base, rows_per_wg, idx, m, n)) {
            pre.before[pass] = to_f32<TC>(C[(int64_t)m * ldc + n]);
            if (link.next_w) pre.next_w[pass] = link.next_w[n];
        }
    }
    return pre;
}

// What the waves of a skinny product's workgroup have summed over their shares of K comes together
// here: through LDS (red: a wave's NT * MT * 256 floats start wave_stride floats apart), in a fixed
// order, then the epilogue.  Called by all threads.
template <int MT, int NT, int WAVES, int EPI, typename TC>
__device__ __forceinline__ void skinny_finish(f32x4 (&acc)[NT][MT], float* red, int wave_stride, TC* __restrict__ C, int M, int N,
                                              int64_t ldc, const NormLink& link, float link_mine,
                                              float (&link_scratch)[WAVES * 64], float (&link_scale)[16], int n_base,
                                              int rows_per_wg, const SkinnyValues<MT, NT, WAVES, EPI>& pre) {
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    // reduce over the waves
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[(size_t)wave * wave_stride + ((t * MT + u) * 4 + r) * 64 + lane] = acc[t][u][r];
    __syncthreads();
    row_scale_finish<WAVES * 64>(link, link_mine, 16, link_scratch, link_scale);
    float next_sq = 0.f;                // producer side: x^2 of the value this thread finishes (one pass only)
#pragma unroll
    for (int pass = 0; pass < pre.PASSES; ++pass) {
        int idx, m, n;
        if (!pre.place(pass, M, N, n_base, rows_per_wg, idx, m, n)) continue;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            s0 += red[(size_t)w * wave_stride + idx];
            if (EPI == 2) s1 += red[(size_t)w * wave_stride + idx + 64];
        }
        if (link.ssq) {
            s0 *= link_scale[m];
            s1 *= link_scale[m];
        }
        if (EPI == 2) {
            C[(int64_t)m * ldc + n / 2] = from_f32<TC>(silu_mul(s0, s1));
        } else if (EPI == 1) {
            const float x = pre.before[pass] + s0;
            C[(int64_t)m * ldc + n] = from_f32<TC>(x);
            if (link.next_w) {
                link.next_h[(int64_t)m * ldc + n] = f32_to_bf16_bits(x * pre.next_w[pass]);
                next_sq = x * x;
            }
        } else {
            C[(int64_t)m * ldc + n] = from_f32<TC>(s0);
        }
    }
    if (EPI == 1 && MT == 1 && NT * 4 <= WAVES && link.next_w) {
        // Every thread of the first 4 NT waves has finished one value (the loop above ran once for
        // it).  Tile t's 16 columns of every row: lanes l, l+16, l+32, l+48 of waves 4t .. 4t+3 hold
        // them (r = wave % 4); rows past M and columns past N added nothing.  One share of the sums
        // per tile of 16 columns: share blockIdx.x * NT + t (the workgroup has 16 NT rows).
        next_sq += __shfl_xor(next_sq, 16, WAVE);
        next_sq += __shfl_xor(next_sq, 32, WAVE);
        __syncthreads();                    // link_scratch may still be read as the consumer's
        if (wave < 4 * NT && lane < 16) link_scratch[wave * 16 + lane] = next_sq;
        __syncthreads();
        if (threadIdx.x < 16 * NT) {
            const int t = threadIdx.x / 16, m = threadIdx.x % 16;
            const float* part = link_scratch + t * 64 + m;
            link.next_ssq[((size_t)blockIdx.x * NT + t) * link.rows + m] = part[0] + part[16] + part[32] + part[48];
        }
    }
}

template <int MT, int NT, int WAVES, int EPI, typename TC>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
                                                                 const bf16_t* __restrict__ W,
                                                                 TC* __restrict__ C, int M, int N, int K,
                                                                 int64_t lda, int64_t ldw, int64_t ldc, NormLink link,
                                                                 int rows_per_wg) {
    extern __shared__ float red[];      // [WAVES][NT][MT][4][64]
    __shared__ float link_scratch[WAVES * 64], link_scale[16];
    const float link_mine = row_scale_begin<WAVES * 64>(link, M, 0, 16);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int r16 = lane % 16, q = lane / 16;
    // A workgroup takes rows_per_wg weight rows (at most 16 * NT): a number that need not fill
    // its last tile of 16, so that the host can size the launch to the CUs.  Lanes of rows it does
    // not have read its last row again, which costs no traffic, and their sums are not stored.
    const int n_base = blockIdx.x * rows_per_wg;
    const auto pre = skinny_prefetch<MT, NT, WAVES, EPI, TC>(C, M, N, ldc, link, n_base, rows_per_wg);

    const bf16_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wrow[t] = W + (int64_t)min(n_base + min(t * 16 + r16, rows_per_wg - 1), N - 1) * ldw;
    const bf16_t* arow[MT];
    bool mvalid[MT];
#pragma unroll
    for (int u = 0; u < MT; ++u) {
        const int m = u * 16 + r16;
        mvalid[u] = m < M;
        arow[u] = A + (int64_t)(mvalid[u] ? m : 0) * lda;
    }
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u) acc[t][u] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Two register buffers: the loads of a wave's next step are in flight while the MFMAs of
    // the current one run.  Loads in the main loop carry no predicate (a predicate makes the
    // compiler fence every load): rows m >= M read row 0 and their results are never stored;
    // the K tail, if any, is a separate last step.
    const int n_full = K / SK_KSTEP;
    bf16x8 wv[2][NT][4], av[2][MT][4];
    auto fetch = [&](int buf, int s) {
        // load j of a step reads, of every row, the 64 contiguous bytes at 64*j: the four quarter
        // lanes of a row take 16 bytes each
        const int k0 = s * SK_KSTEP + q * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int t = 0; t < NT; ++t) wv[buf][t][j] = load_chunk(wrow[t] + k0 + 32 * j);
#pragma unroll
            for (int u = 0; u < MT; ++u)
                av[buf][u][j] = load_chunk(arow[u] + k0 + 32 * j);
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int u = 0; u < MT; ++u)
                    acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[buf][t][j], av[buf][u][j], acc[t][u], 0, 0, 0);
    };
    int s = wave;
    if (s < n_full) fetch(0, s);
    while (s < n_full) {
        if (s + WAVES < n_full) fetch(1, s + WAVES);
        multiply(0);
        s += WAVES;
        if (s >= n_full) break;
        if (s + WAVES < n_full) fetch(0, s + WAVES);
        multiply(1);
        s += WAVES;
    }
    if (K % SK_KSTEP != 0 && wave == n_full % WAVES) {
        const int k0 = n_full * SK_KSTEP + q * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + 32 * j;
            const bool kvalid = k < K;
#pragma unroll
            for (int t = 0; t < NT; ++t) wv[0][t][j] = kvalid ? load_chunk(wrow[t] + k) : zero_chunk();
#pragma unroll
            for (int u = 0; u < MT; ++u) av[0][u][j] = kvalid ? load_chunk(arow[u] + k) : zero_chunk();
        }
        multiply(0);
    }
    skinny_finish<MT, NT, WAVES, EPI, TC>(acc, red, NT * MT * 4 * 64, C, M, N, ldc, link, link_mine, link_scratch, link_scale, n_base,
                                          rows_per_wg, pre);
}

// ---- skinny, weights and activations staged through LDS -----------------------------------------
// The same division of work (a workgroup takes a few weight rows, its eight waves take K in turns
// of 64, up to 16 activation rows), but a wave's loads go from global memory straight into LDS, a
// kilobyte each (eight rows by 128 bytes: whole lines), into stages of the wave's own; the MFMA
// operands are read from there.  Whole lines are what lets the weights be marked non-temporal
// (the kernel above asks for 64 bytes of 16 rows at a time, which such loads make slower), and
// stages in LDS cost no registers, so that several steps of a wave are in flight: with 16 weight
// rows and up to 8 activation rows six stages of 3 KB (and with 48 and 16, two of 8 KB, which
// still beat the kernel above: 12,288 x 4,096 at 16 rows 18.5 against 22.2 us).  No barrier in the loop: a wave reads only
// what it loaded, when its own count of outstanding loads says that it has arrived.  All loads of
// the loop are assembly for that count's sake, as in the tile kernel.
#define SKS_KSTEP 64
#define SKS_LDS_BYTES (160 * 1024)
// s_waitcnt vmcnt(n) for a number known only at run time (the same in every lane)
__device__ __forceinline__ void wait_for_loads_upto(int n) {
    switch (n) {
#define SKS_CASE(i) case i: wait_for_loads<i>(); break;
        SKS_CASE(0) SKS_CASE(1) SKS_CASE(2) SKS_CASE(3) SKS_CASE(4) SKS_CASE(5) SKS_CASE(6) SKS_CASE(7)
        SKS_CASE(8) SKS_CASE(9) SKS_CASE(10) SKS_CASE(11) SKS_CASE(12) SKS_CASE(13) SKS_CASE(14) SKS_CASE(15)
        SKS_CASE(16) SKS_CASE(17) SKS_CASE(18) SKS_CASE(19) SKS_CASE(20) SKS_CASE(21) SKS_CASE(22) SKS_CASE(23)
        SKS_CASE(24) SKS_CASE(25) SKS_CASE(26) SKS_CASE(27) SKS_CASE(28) SKS_CASE(29) SKS_CASE(30) SKS_CASE(31)
        SKS_CASE(32) SKS_CASE(33) SKS_CASE(34) SKS_CASE(35) SKS_CASE(36) SKS_CASE(37) SKS_CASE(38) SKS_CASE(39)
        SKS_CASE(40) SKS_CASE(41) SKS_CASE(42)
#undef SKS_CASE
        default: wait_for_loads<0>(); break;
    }
}

template <int NT, int EPI, typename TC>
__global__ __launch_bounds__(512) void gemm_skinny_staged_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                                 TC* __restrict__ C, int M, int N, int K, int64_t lda,
                                                                 int64_t ldw, int64_t ldc, NormLink link, int rows_per_wg,
                                                                 int n_stages) {
    extern __shared__ __attribute__((aligned(1024))) char staged_lds[];
    __shared__ float link_scratch[512], link_scale[16];
    const float link_mine = row_scale_begin<512>(link, M, 0, 16);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const int r16 = lane % 16, q = lane / 16;
    const int n_base = blockIdx.x * rows_per_wg;
    const auto pre = skinny_prefetch<1, NT, 8, EPI, TC>(C, M, N, ldc, link, n_base, rows_per_wg);
    // kilobytes (loads of a wave) that a step brings in: eight weight rows each, eight activation rows each
    const int w_loads = (rows_per_wg + 7) / 8, a_loads = (M + 7) / 8;
    const int stage_bytes = (w_loads + a_loads) * 1024;
    const unsigned lds_wave = __builtin_amdgcn_readfirstlane(
        (unsigned)(size_t)(__attribute__((address_space(3))) char*)staged_lds + wave * (n_stages * stage_bytes));
    const char* my_lds = staged_lds + wave * (n_stages * stage_bytes);
    // Load i of the weights fills LDS rows 8i .. 8i+7 of the stage, 128 bytes a row; the lane that
    // fills 16-byte slot p of a row fetches the chunk that belongs there (slots are XORed with the
    // row, so that the 16 rows an MFMA operand is read from lie in different banks).  Rows that
    // the workgroup or the matrix does not have repeat its last one and are never stored.
    const int lrow = lane / 8, lslot = lane % 8;
    unsigned w_off[2 * NT], a_off[2];
#pragma unroll
    for (int i = 0; i < 2 * NT; ++i) {
        const int row = 8 * i + lrow;
        const int grow = min(n_base + min(row, rows_per_wg - 1), N - 1) - n_base;
        w_off[i] = (unsigned)((grow * ldw + (lslot ^ ((row >> 1) & 7)) * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = 8 * i + lrow;
        a_off[i] = (unsigned)((min(row, M - 1) * lda + (lslot ^ ((row >> 1) & 7)) * 8) * 2);
    }
    const bf16_t* w_rows = W + (int64_t)n_base * ldw;
    // step k of this wave is K's slice wave + 8 k
    const int n_slices = K / SKS_KSTEP;
    const int n_mine = wave < n_slices ? (n_slices - wave + 7) / 8 : 0;
    auto issue = [&](int k) {
        const unsigned to = lds_wave + (k % n_stages) * stage_bytes;
        const int k0 = (wave + 8 * k) * SKS_KSTEP;
        const void* wsrc = same_in_every_lane(w_rows + k0);
        const void* asrc = same_in_every_lane(A + k0);
#pragma unroll
        for (int i = 0; i < 2 * NT; ++i)
            if (i < w_loads) stream_16_bytes_to_lds(w_off[i], wsrc, to + i * 1024);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            if (i < a_loads) load_16_bytes_to_lds(a_off[i], asrc, to + (w_loads + i) * 1024);
    };
    f32x4 acc[NT][1];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    // where this lane's operands lie in a stage: weight row 16 t + r16 and activation row r16 (rows
    // that were not loaded repeat loaded ones: their results are never stored), chunk 4 j + q
    int w_at[NT][2], a_at[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int row = (16 * t + r16) % (8 * w_loads);
            w_at[t][j] = row * 128 + (((4 * j + q) ^ ((row >> 1) & 7)) * 16);
        }
        const int row = r16 % (8 * a_loads);
        a_at[j] = w_loads * 1024 + row * 128 + (((4 * j + q) ^ ((row >> 1) & 7)) * 16);
    }
    const int per_step = w_loads + a_loads;
    for (int k = 0; k < min(n_stages, n_mine); ++k) issue(k);
    for (int k = 0; k < n_mine; ++k) {
        // the steps asked for after this one may still be on their way
        wait_for_loads_upto(min(n_stages - 1, n_mine - 1 - k) * per_step);
        __builtin_amdgcn_sched_barrier(0);
        const char* st = my_lds + (k % n_stages) * stage_bytes;
        bf16x8 wf[NT][2], af[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            af[j] = *(const bf16x8*)(st + a_at[j]);
#pragma unroll
            for (int t = 0; t < NT; ++t) wf[t][j] = *(const bf16x8*)(st + w_at[t][j]);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t][j], af[j], acc[t][0], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        // the stage is read out (the products above waited for its operands): it takes step k + n_stages
        if (k + n_stages < n_mine) issue(k + n_stages);
    }
    // each wave leaves its sums in its own stages, which only it has read
    skinny_finish<1, NT, 8, EPI, TC>(acc, (float*)staged_lds, n_stages * stage_bytes / 4, C, M, N, ldc, link, link_mine, link_scratch,
                                     link_scale, n_base, rows_per_wg, pre);
}

// Whether the staged kernel takes a product, and with how many stages a wave.
// two_a_cu: half of the LDS, so that two workgroups share a CU
static int skinny_staged_stages(int M, int K, int rows_per_wg, bool two_a_cu = false) {
    if (M > 16 || K % SKS_KSTEP || rows_per_wg % 8 || rows_per_wg > 48) return 0;
    const int per_step = (rows_per_wg + 7) / 8 + (M + 7) / 8;
    int stages = ((two_a_cu ? SKS_LDS_BYTES / 2 : SKS_LDS_BYTES) - 4096) / 8 / (per_step * 1024);      // (the kernel has 2 KB of its own)
    if (stages > 8) stages = 8;
    while (stages > 1 && (stages - 1) * per_step > 42) --stages;
    return stages >= 2 ? stages : 0;
}
template <int NT>
static int launch_skinny_staged(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                int64_t ldw, int64_t ldc, int epi, hipStream_t stream, NormLink link, int rows_per_wg) {
    const int stages = skinny_staged_stages(M, K, rows_per_wg, ceil_div(N, rows_per_wg) > n_compute_units());
    PICOLM_REQUIRE(stages > 0 && rows_per_wg <= 16 * NT, "gemm_skinny: the staged kernel does not take M=%d K=%d with %d rows a workgroup", M, K, rows_per_wg);
    PICOLM_REQUIRE(!link.next_w || (NT <= 2 && epi == 1 && rows_per_wg == 16 * NT && link.next_parts >= ceil_div(N, 16)),
                   "gemm_skinny: whole tiles of 16 weight rows with the accumulating epilogue prepare a norm");
    PICOLM_REQUIRE((!link.ssq && !link.next_w) || link.rows == 16, "gemm_skinny: a split norm goes with up to 16 rows here");
    PICOLM_REQUIRE(64 * ldw * 2 < (1ll << 31) && 16 * lda * 2 < (1ll << 31), "gemm_skinny: row strides %lld / %lld overflow 32-bit offsets",
                   (long long)lda, (long long)ldw);
    dim3 grid(ceil_div(N, rows_per_wg)), block(512);
    const size_t lds = (size_t)8 * stages * ((rows_per_wg + 7) / 8 + (M + 7) / 8) * 1024;
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
#define SKS_LAUNCH(EPI, TC)                                                                                   \
    {                                                                                                         \
        static bool raised = false;                                                                           \
        if (!raised) {                                                                                        \
            hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_staged_kernel<NT, EPI, TC>,            \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, SKS_LDS_BYTES - 4096); \
            PICOLM_REQUIRE(e == hipSuccess, "gemm_skinny: cannot raise the LDS limit: %s", hipGetErrorString(e)); \
            raised = true;                                                                                    \
        }                                                                                                     \
        gemm_skinny_staged_kernel<NT, EPI, TC><<<grid, block, lds, stream>>>(a, w, (TC*)C, M, N, K, lda, ldw, ldc, link, \
                                                                            rows_per_wg, stages);            \
    }
    if (epi == 0 && c_dt == PICOLM_F32) SKS_LAUNCH(0, float)
    else if (epi == 0 && c_dt == PICOLM_BF16) SKS_LAUNCH(0, bf16_t)
    else if (epi == 1 && c_dt == PICOLM_F32) SKS_LAUNCH(1, float)
    else if (epi == 2 && c_dt == PICOLM_BF16) SKS_LAUNCH(2, bf16_t)
    else if (epi == 2 && c_dt == PICOLM_F32) SKS_LAUNCH(2, float)
    else PICOLM_REQUIRE(false, "gemm_skinny: unsupported epilogue %d with output dtype %d", epi, c_dt);
#undef SKS_LAUNCH
    PICOLM_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

template <int MT, int NT, int WAVES>
static int launch_skinny(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                         int64_t ldw, int64_t ldc, int epi, hipStream_t stream, NormLink link = NormLink{},
                         int rows_per_wg = 16 * NT) {
    PICOLM_REQUIRE(!link.next_w || (MT == 1 && NT == 1 && WAVES == 8 && epi == 1 && link.next_parts >= ceil_div(N, 16)),
                   "gemm_skinny: only the 16x16 tile with the accumulating epilogue prepares a norm");
    PICOLM_REQUIRE((!link.ssq && !link.next_w) || (M <= 16 && link.rows == 16),
                   "gemm_skinny: a split norm goes with up to 16 rows here, got %d", M);
    PICOLM_REQUIRE(rows_per_wg >= 2 && rows_per_wg <= 16 * NT && rows_per_wg % 2 == 0 && (!link.next_w || rows_per_wg == 16),
                   "gemm_skinny: %d weight rows a workgroup do not fit %d tiles of 16", rows_per_wg, NT);
    dim3 grid(ceil_div(N, rows_per_wg)), block(WAVES * 64);
    const size_t lds = sizeof(float) * WAVES * NT * MT * 4 * 64;
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
#define SK_LAUNCH(EPI, TC)                                                                              \
    {                                                                                                   \
        static size_t raised = 48 * 1024;                                                               \
        if (lds > raised) {                                                                             \
            hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, NT, WAVES, EPI, TC>, \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);   \
            PICOLM_REQUIRE(e == hipSuccess, "gemm_skinny: cannot raise the LDS limit: %s",              \
                           hipGetErrorString(e));                                                       \
            raised = lds;                                                                               \
        }                                                                                               \
        gemm_skinny_kernel<MT, NT, WAVES, EPI, TC><<<grid, block, lds, stream>>>(a, w, (TC*)C, M, N, K, lda, ldw, ldc, link, rows_per_wg); \
    }
    if (epi == 0 && c_dt == PICOLM_F32) SK_LAUNCH(0, float)
    else if (epi == 0 && c_dt == PICOLM_BF16) SK_LAUNCH(0, bf16_t)
    else if (epi == 1 && c_dt == PICOLM_F32) SK_LAUNCH(1, float)
    else if (epi == 2 && c_dt == PICOLM_BF16) SK_LAUNCH(2, bf16_t)
    else if (epi == 2 && c_dt == PICOLM_F32) SK_LAUNCH(2, float)
    else PICOLM_REQUIRE(false, "gemm_skinny: unsupported epilogue %d with output dtype %d", epi, c_dt);
#undef SK_LAUNCH
    PICOLM_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

// variant: 0 picks by shape; 1..6 name (MT,NT,WAVES) combinations for tuning and tests, 9 is 1 without the staged kernel
// Weight rows a workgroup of the 16-row kernel takes: 16, or, where the workgroups of that size
// would leave a last round of the CUs mostly empty, the multiple of 8 up to 64 with which the
// launch takes the fewest rows per CU (6144 rows on 256 CUs: 24 rows each instead of 16 in one
// and a half rounds).
static int skinny_rows_per_wg(int N, int M) {
    const int cus = n_compute_units();
    int best = 16;
    int64_t best_cost = (int64_t)ceil_div(ceil_div(N, 16), cus) * 16 * 4;
    for (int rows = 24; rows <= 64; rows += 8) {
        // rounds of the CUs times what a workgroup moves; the rows that its last tile reads a
        // second time cost no memory traffic but a quarter of their share of load instructions
        const int padded = (rows + 15) / 16 * 16;
        const int64_t cost = (int64_t)ceil_div(ceil_div(N, rows), cus) * (4 * rows + (padded - rows));
        // as cheap with fewer, larger workgroups: every workgroup reads all the activations, so with
        // many rows the fewer win (12288 x 4096: 22 against 26 us at 16 rows), with one row the more
        // (20 against 22 us)
        // (and one round of up to 32 rows a workgroup suits the staged kernel; with 48 rows it has
        // three stages and is no better than two rounds of the other: 12288 x 4096, 21 against 19 us)
        if (cost < best_cost || (cost == best_cost && (M > 8 || (rows <= 32 && ceil_div(N, rows) <= cus)))) {
            best = rows;
            best_cost = cost;
        }
    }
    return best;
}
template <int MT>
static int launch_skinny_sized(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                               int64_t ldw, int64_t ldc, int epi, hipStream_t stream, NormLink link, bool staged = true) {
    // a product that prepares a norm leaves one share of its sums per 16 weight rows, so its
    // workgroups take whole tiles: 16 rows, or 32 where that makes one round of the CUs out of two
    const int cus = n_compute_units();
    const bool two_tiles = N % 32 == 0 && ceil_div(N, 16) > cus && N / 32 <= cus && skinny_staged_stages(M, K, 32) > 0;
    const int rows = link.next_w ? (staged && MT == 1 && two_tiles ? 32 : 16) : skinny_rows_per_wg(N, M);
    // A launch of more workgroups than CUs gets half the LDS a workgroup, so that two share a CU and
    // one's start and end overlap the other's loop (with all of it, a second round of workgroups
    // waits for the first to leave: 12,288 rows as 512 workgroups took 22 us, 17.4 this way and 19
    // in the kernel above; a vocabulary of 128,256 rows 183, 155 and 165).
    if (staged && MT == 1 && skinny_staged_stages(M, K, rows, ceil_div(N, rows) > n_compute_units()) > 0) {
        if (rows <= 16) return launch_skinny_staged<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
        if (rows <= 32) return launch_skinny_staged<2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
        return launch_skinny_staged<3>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
    }
    if (rows <= 16) return launch_skinny<MT, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
    if (rows <= 32) return launch_skinny<MT, 2, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
    if (rows <= 48) return launch_skinny<MT, 3, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
    return launch_skinny<MT, 4, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epi, stream, link, rows);
}

extern "C" int picolm_gemm_skinny(const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                  int64_t lda, int64_t ldw, int64_t ldc, int epilogue, int variant,
                                  hipStream_t stream) {
    if (check_mfma_operands("gemm_skinny", A, W, M, N, K, lda, ldw, ldc, epilogue, c_dt)) return -1;
    PICOLM_REQUIRE(M <= 64, "gemm_skinny: M=%d exceeds 64", M);
    if (M == 0) return 0;
    if (variant == 0) variant = M <= 16 ? 1 : (M <= 32 ? 3 : (N >= 8192 ? 6 : 5));
    switch (variant) {
        case 1: return launch_skinny_sized<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, NormLink{});
        case 9: return launch_skinny_sized<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, NormLink{}, false);   // never staged
        case 8: return launch_skinny<1, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);      // 16 rows a workgroup
        case 2: return launch_skinny<1, 2, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 3: return launch_skinny<2, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 4: return launch_skinny<2, 2, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 5: return launch_skinny<4, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 6: return launch_skinny<4, 2, 4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
    }
    PICOLM_REQUIRE(false, "gemm_skinny: unknown variant %d", variant);
}

// The skinny side of picolm_gemm_linked (up to 16 rows).
int picolm_gemm_skinny_linked_(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                               int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link) {
    if (variant == 0 || variant == 1) return launch_skinny_sized<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, link);
    PICOLM_REQUIRE(false, "gemm_linked: skinny variant %d cannot take part in a split norm", variant);
}
