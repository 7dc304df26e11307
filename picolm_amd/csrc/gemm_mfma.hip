// bf16 x bf16 -> float products on the matrix cores of gfx950: C[M,N] = A[M,K] * W[N,K]^T.
//
// The skinny kernel feeds the weight tile as the MFMA's first operand and the activation tile
// as its second, so an accumulator lane holds four consecutive output columns n of one row m
// and gate/up pairs of the row-interleaved gated layout meet in one lane.
//
//   skinny (M <= 64, the decode step): HBM-bound.  A wave streams 16*NT weight rows straight
//     from global memory into MFMA operand registers, 16 bytes a lane; the waves of a block
//     split K between them and reduce through LDS.  Every weight byte is read once.
//   tiled (M > 64, the prefill step): block tiles of 128x128 to 256x256 in LDS with an XOR swizzle
//     of 16-byte chunks, 32x32x16 MFMAs; here the activation tile is the first operand, so that
//     stores are whole 128-byte runs.  Tiles reach LDS straight from global memory
//     (global_load_lds) when K is a multiple of 64, else through staging registers.  These
//     kernels are bound by what L2 delivers to the CUs, not by the matrix cores.
//
// The order of the K summation inside an MFMA does not matter, so a lane's 8-element chunk
// may come from any K offset as long as both operands use the same offset.
#include <type_traits>
#include "common.h"
#include "api.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ bf16x8 load_chunk(const bf16_t* p) { return *(const bf16x8*)p; }
__device__ __forceinline__ bf16x8 zero_chunk() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
    return z;
}
__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// =============================================================================================
// a norm split between two products
// =============================================================================================
// In a decode step an RMSNorm of a few rows is all launch latency.  It can ride on the products
// around it instead: the product that finishes the rows of the residual stream (epilogue 1) also
// leaves, for the norm that follows, next_h = bf16(x * w) and one partial sum of x^2 per row and
// workgroup; the product that consumes the normed rows takes next_h as its input and multiplies its
// sums by 1 / sqrt(sum(x^2) / len + eps) in float.  Both sides only for up to 16 rows.
struct NormLink {
    const float* next_w;    // producer: weights of the norm that follows [N], or null
    bf16_t* next_h;         //   [M][ld of C] what the next product reads
    float* next_ssq;        //   [next_parts][rows] partial sums of x^2, one row per workgroup
    int next_parts;
    const float* ssq;       // consumer: the partial sums a producer left [n_parts][rows], or null
    int n_parts;
    float inv_len, eps;     //   1 / row length of the norm, its eps
    int rows;               // 16 (products of up to 16 rows) or 64: rows that the sums are kept for
};

// Consumer side.  `begin` has every thread ask for its share of the partial sums (row
// m0 + tid % tile_rows, every (THREADS/tile_rows)-th part) before the main loop; `finish` adds
// them up in a fixed order and leaves the factors of the tile's rows in LDS.  Both are called by
// all THREADS threads of the workgroup; tile_rows is a power of two of at most THREADS.
template <int THREADS>
__device__ __forceinline__ float row_scale_begin(const NormLink& k, int M, int m0, int tile_rows) {
    float mine = 0.f;
    if (k.ssq) {
        const int m = m0 + threadIdx.x % tile_rows, stride = THREADS / tile_rows;
        if (m < M) {
            // eight loads are asked for before the first is added: one trip to memory, not eight
            for (int p0 = threadIdx.x / tile_rows; p0 < k.n_parts; p0 += 8 * stride) {
                float v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = k.ssq[(size_t)min(p0 + i * stride, k.n_parts - 1) * k.rows + m];
#pragma unroll
                for (int i = 0; i < 8; ++i) mine += p0 + i * stride < k.n_parts ? v[i] : 0.f;
            }
        }
    }
    return mine;
}
template <int THREADS, int SCALES>
__device__ __forceinline__ void row_scale_finish(const NormLink& k, float mine, int tile_rows, float (&scratch)[THREADS],
                                                 float (&scale)[SCALES]) {
    if (!k.ssq) return;          // uniform over the workgroup
    scratch[threadIdx.x] = mine;             // [share][row of the tile]
    __syncthreads();
    if ((int)threadIdx.x < tile_rows) {
        float total = 0.f;
        for (int g = 0; g < THREADS / tile_rows; ++g) total += scratch[g * tile_rows + threadIdx.x];
        scale[threadIdx.x] = 1.0f / sqrtf(total * k.inv_len + k.eps);
    }
    __syncthreads();
}

// =============================================================================================
// skinny
// =============================================================================================
#define SK_KSTEP 128      // K elements one wave consumes per step: 4 MFMAs of 32

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
    // reduce over the waves
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[(((wave * NT + t) * MT + u) * 4 + r) * 64 + lane] = acc[t][u][r];
    __syncthreads();
    row_scale_finish<WAVES * 64>(link, link_mine, 16, link_scratch, link_scale);
    constexpr int PER_WAVE = NT * MT * 4 * 64;
    constexpr int STEP = (EPI == 2) ? 2 : 1;
    float next_sq = 0.f;                // producer side: x^2 of the value this thread finishes (MT = NT = 1 only)
    // value v = ((t*MT + u)*4 + r)*64 + l ; the gated epilogue takes r and r+1 together
    for (int v = threadIdx.x; v < PER_WAVE / STEP; v += WAVES * 64) {
        int l, r, tu;
        if (EPI == 2) {
            l = v % 64;
            r = 2 * ((v / 64) % 2);
            tu = v / 128;
        } else {
            l = v % 64;
            r = (v / 64) % 4;
            tu = v / 256;
        }
        const int u = tu % MT, t = tu / MT;
        const int idx = ((t * MT + u) * 4 + r) * 64 + l;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            s0 += red[w * PER_WAVE + idx];
            if (EPI == 2) s1 += red[w * PER_WAVE + idx + 64];
        }
        const int n = n_base + t * 16 + 4 * (l / 16) + r;
        const int m = u * 16 + l % 16;
        if (m >= M || n >= N || t * 16 + 4 * (l / 16) + r >= rows_per_wg) continue;
        if (link.ssq) {
            s0 *= link_scale[m];
            s1 *= link_scale[m];
        }
        if (EPI == 2) {
            C[(int64_t)m * ldc + n / 2] = from_f32<TC>(silu_mul(s0, s1));
        } else if (EPI == 1) {
            TC* p = C + (int64_t)m * ldc + n;
            const float x = to_f32<TC>(*p) + s0;
            *p = from_f32<TC>(x);
            if (link.next_w) {
                link.next_h[(int64_t)m * ldc + n] = f32_to_bf16_bits(x * link.next_w[n]);
                next_sq = x * x;
            }
        } else {
            C[(int64_t)m * ldc + n] = from_f32<TC>(s0);
        }
    }
    if (EPI == 1 && MT == 1 && NT == 1 && link.next_w) {
        // this workgroup's 16 columns of every row: lanes l, l+16, l+32, l+48 of the first four
        // waves hold them (r = wave); rows past M and columns past N added nothing
        next_sq += __shfl_xor(next_sq, 16, WAVE);
        next_sq += __shfl_xor(next_sq, 32, WAVE);
        __syncthreads();                    // link_scratch may still be read as the consumer's
        if (wave < 4 && lane < 16) link_scratch[wave * 16 + lane] = next_sq;
        __syncthreads();
        if (threadIdx.x < 16)
            link.next_ssq[(size_t)blockIdx.x * link.rows + threadIdx.x] =
                link_scratch[threadIdx.x] + link_scratch[16 + threadIdx.x] + link_scratch[32 + threadIdx.x] + link_scratch[48 + threadIdx.x];
    }
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

// ---- skinny, with the activations resident ---------------------------------------------------
// For M <= 16 and K <= STEPS * 1024: a wave keeps the activation chunks of its K slices in
// registers for the whole launch and a workgroup walks over many tiles of 16 weight rows, with
// the next tile's weights in flight while the current one is multiplied and reduced.  The
// activations are read once per workgroup instead of once per tile, and the gap between tiles
// (the reduction through LDS, the epilogue) no longer leaves the memory pipe empty.
template <int STEPS, int EPI, typename TC>
__global__ __launch_bounds__(512) void gemm_skinny_resident_kernel(const bf16_t* __restrict__ A,
                                                                   const bf16_t* __restrict__ W,
                                                                   TC* __restrict__ C, int M, int N, int K,
                                                                   int64_t lda, int64_t ldw, int64_t ldc, NormLink link) {
    constexpr int WAVES = 8;
    __shared__ float red[2][WAVES][4][64];
    __shared__ float link_scratch[WAVES * 64], link_scale[16];
    const float link_mine = row_scale_begin<WAVES * 64>(link, M, 0, 16);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int r16 = lane % 16, q = lane / 16;
    const int n_full = K / SK_KSTEP;            // K is a whole number of steps (the host sees to that)
    const int n_tiles = (N + 15) / 16;

    bf16x8 av[STEPS][4];
    int koff[STEPS];                            // element offset of this lane's first chunk of step i
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        const int s = wave + i * WAVES;
        const bool valid = s < n_full && r16 < M;
        koff[i] = min(s, n_full - 1) * SK_KSTEP + q * 8;      // a step past the end reads the last one; its activations are zero
#pragma unroll
        for (int j = 0; j < 4; ++j)
            av[i][j] = valid ? load_chunk(A + (int64_t)r16 * lda + koff[i] + 32 * j) : zero_chunk();
    }
    auto fetch = [&](bf16x8 (&wv)[STEPS][4], int tile) {
        const bf16_t* wrow = W + (int64_t)min(tile * 16 + r16, N - 1) * ldw;
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[i][j] = load_chunk(wrow + koff[i] + 32 * j);
    };
    auto finish = [&](const bf16x8 (&wv)[STEPS][4], int tile, int buf) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i][j], av[i][j], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) red[buf][wave][r][lane] = acc[r];
        __syncthreads();
        // value (r, l): n = 16*tile + 4*(l/16) + r, m = l%16; the gated epilogue takes r and r+1 together
        constexpr int STEP = (EPI == 2) ? 2 : 1;
        const int v = threadIdx.x;
        if (v < 256 / STEP) {
            const int l = v % 64, r = EPI == 2 ? 2 * (v / 64) : v / 64;
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                s0 += red[buf][w][r][l];
                if (EPI == 2) s1 += red[buf][w][r + 1][l];
            }
            const int n = tile * 16 + 4 * (l / 16) + r, m = l % 16;
            if (m < M && n < N) {
                if (link.ssq) {
                    s0 *= link_scale[m];
                    s1 *= link_scale[m];
                }
                if (EPI == 2) {
                    C[(int64_t)m * ldc + n / 2] = from_f32<TC>(silu_mul(s0, s1));
                } else if (EPI == 1) {
                    TC* p = C + (int64_t)m * ldc + n;
                    *p = from_f32<TC>(to_f32<TC>(*p) + s0);
                } else {
                    C[(int64_t)m * ldc + n] = from_f32<TC>(s0);
                }
            }
        }
    };
    // two register sets of weights and two LDS buffers alternate, so that one barrier a tile is
    // enough; tiles past the end read the last tile again and are not finished
    bf16x8 w0[STEPS][4], w1[STEPS][4];
    const int stride = gridDim.x;
    int tile = blockIdx.x;
    fetch(w0, min(tile, n_tiles - 1));
    row_scale_finish<WAVES * 64>(link, link_mine, 16, link_scratch, link_scale);
    while (tile < n_tiles) {
        fetch(w1, min(tile + stride, n_tiles - 1));
        __builtin_amdgcn_sched_barrier(0);      // the next tile is asked for before this one is waited for
        finish(w0, tile, 0);
        tile += stride;
        if (tile >= n_tiles) break;
        fetch(w0, min(tile + stride, n_tiles - 1));
        __builtin_amdgcn_sched_barrier(0);
        finish(w1, tile, 1);
        tile += stride;
    }
}

template <int STEPS>
static int launch_skinny_resident(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                  int64_t ldw, int64_t ldc, int epi, hipStream_t stream, NormLink link = NormLink{}) {
    PICOLM_REQUIRE(!link.next_w, "gemm_skinny: the resident variant prepares no norm");
    PICOLM_REQUIRE(!link.ssq || link.rows == 16, "gemm_skinny: a split norm goes with up to 16 rows here");
    PICOLM_REQUIRE(M <= 16 && K % SK_KSTEP == 0 && K <= STEPS * 8 * SK_KSTEP,
                   "gemm_skinny: the resident variant takes M <= 16 and K a multiple of %d up to %d, got M=%d K=%d",
                   SK_KSTEP, STEPS * 8 * SK_KSTEP, M, K);
    // one workgroup a CU; the same number of tiles for every workgroup where that is possible
    const int n_tiles = ceil_div(N, 16);
    const int rounds = ceil_div(n_tiles, 256);
    dim3 grid(ceil_div(n_tiles, rounds)), block(512);
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
#define SR_LAUNCH(EPI, TC) \
    gemm_skinny_resident_kernel<STEPS, EPI, TC><<<grid, block, 0, stream>>>(a, w, (TC*)C, M, N, K, lda, ldw, ldc, link);
    if (epi == 0 && c_dt == PICOLM_F32) SR_LAUNCH(0, float)
    else if (epi == 0 && c_dt == PICOLM_BF16) SR_LAUNCH(0, bf16_t)
    else if (epi == 1 && c_dt == PICOLM_F32) SR_LAUNCH(1, float)
    else if (epi == 2 && c_dt == PICOLM_BF16) SR_LAUNCH(2, bf16_t)
    else if (epi == 2 && c_dt == PICOLM_F32) SR_LAUNCH(2, float)
    else PICOLM_REQUIRE(false, "gemm_skinny: unsupported epilogue %d with output dtype %d", epi, c_dt);
#undef SR_LAUNCH
    PICOLM_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

static int check_mfma_operands(const char* who, const void* A, const void* W, int M, int N, int K, int64_t lda,
                               int64_t ldw, int64_t ldc, int epi, int c_dt) {
    PICOLM_REQUIRE(M >= 0 && N > 0 && K > 0, "%s: bad sizes M=%d N=%d K=%d", who, M, N, K);
    PICOLM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0,
                   "%s: K=%d and the row strides (%lld, %lld) must be multiples of 8", who, K, (long long)lda,
                   (long long)ldw);
    PICOLM_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "%s: operands must be 16-byte aligned", who);
    PICOLM_REQUIRE(epi >= 0 && epi <= 2, "%s: unknown epilogue %d", who, epi);
    PICOLM_REQUIRE(epi != 1 || c_dt == PICOLM_F32, "%s: accumulation needs a float output", who);
    PICOLM_REQUIRE(epi != 2 || N % 2 == 0, "%s: the gated epilogue needs an even N, got %d", who, N);
    PICOLM_REQUIRE(lda >= K && ldw >= K && ldc >= (epi == 2 ? N / 2 : N), "%s: leading dimensions too small", who);
    return 0;
}

// variant: 0 picks by shape; 1..6 name (MT,NT,WAVES) combinations for tuning and tests, 7 is
// the variant with resident activations
// Weight rows a workgroup of the 16-row kernel takes: 16, or, where the workgroups of that size
// would leave a last round of the CUs mostly empty, the multiple of 8 up to 64 with which the
// launch takes the fewest rows per CU (6144 rows on 256 CUs: 24 rows each instead of 16 in one
// and a half rounds).
static int n_compute_units() {
    static int n_cus = 0;
    if (n_cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        n_cus = hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0
                    ? prop.multiProcessorCount : 256;
    }
    return n_cus;
}
static int skinny_rows_per_wg(int N) {
    const int cus = n_compute_units();
    int best = 16;
    int64_t best_cost = (int64_t)ceil_div(ceil_div(N, 16), cus) * 16 * 4;
    for (int rows = 24; rows <= 64; rows += 8) {
        // rounds of the CUs times what a workgroup moves; the rows that its last tile reads a
        // second time cost no memory traffic but a quarter of their share of load instructions
        const int padded = (rows + 15) / 16 * 16;
        const int64_t cost = (int64_t)ceil_div(ceil_div(N, rows), cus) * (4 * rows + (padded - rows));
        if (cost < best_cost) {
            best = rows;
            best_cost = cost;
        }
    }
    return best;
}
template <int MT>
static int launch_skinny_sized(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                               int64_t ldw, int64_t ldc, int epi, hipStream_t stream, NormLink link) {
    const int rows = link.next_w ? 16 : skinny_rows_per_wg(N);
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
    if (variant == 0) {
        // many tiles a CU and several rows: the resident variant reads the activations once and
        // keeps the memory pipe full between tiles (a few rows cost little to re-read, and then
        // several workgroups a CU hide more latency); few tiles: one workgroup a tile
        if (M > 4 && M <= 16 && N >= 16384 && K % SK_KSTEP == 0 && K <= 4 * 8 * SK_KSTEP) variant = 7;
        else variant = M <= 16 ? 1 : (M <= 32 ? 3 : (N >= 8192 ? 6 : 5));
    }
    switch (variant) {
        case 1: return launch_skinny_sized<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, NormLink{});
        case 8: return launch_skinny<1, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);      // 16 rows a workgroup
        case 2: return launch_skinny<1, 2, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 3: return launch_skinny<2, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 4: return launch_skinny<2, 2, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 5: return launch_skinny<4, 1, 8>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 6: return launch_skinny<4, 2, 4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 7: return launch_skinny_resident<4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
    }
    PICOLM_REQUIRE(false, "gemm_skinny: unknown variant %d", variant);
}

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

// =============================================================================================
// tiled, with tiles loaded straight into LDS
// =============================================================================================
// The same block tiles and MFMA layout as above, but global memory is read by
// global_load_lds_dwordx4: a wave's 64 lanes bring 16 bytes each to 1 KB of consecutive LDS, with
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
// A pointer that is the same in every lane, said so that it lies in scalar registers whatever
// the compiler made of the arithmetic that led to it.
__device__ __forceinline__ const void* same_in_every_lane(const void* p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const void*)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void load_16_bytes_to_lds(unsigned byte_offset, const void* base, unsigned lds_address) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(byte_offset), "s"(base), "s"(lds_address)
                 : "memory");
}
template <int N_OUTSTANDING>
__device__ __forceinline__ void wait_for_loads() {      // vmcnt(N), other counters untouched
    static_assert(N_OUTSTANDING < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((N_OUTSTANDING & 15) | (7 << 4) | (15 << 8) | ((N_OUTSTANDING >> 4) << 14));
}

template <int TN, int TM, int WN, int WM, int BK, int NS, int EPI, typename TC>
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
    const int first_step = tiles_m == 1 ? (int)(((unsigned)tile * 5u + blockIdx.y * 3u) % (unsigned)n_steps) : 0;
    auto issue = [&](int stage, int step) {
        const unsigned to = lds_wave + stage * (STAGE * 2);
        step += first_step;
        if (step >= n_steps) step -= n_steps;
        const void* wsrc = same_in_every_lane(w_tile + step * BK);
        const void* asrc = same_in_every_lane(a_tile + step * BK);
#pragma unroll
        for (int j = 0; j < W_LOADS; ++j) load_16_bytes_to_lds(w_off[j], wsrc, to + j * (NW * RG * BK * 2));
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

template <int TN, int TM, int WN, int WM, int BK, int NS>
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
            PICOLM_REQUIRE(e == hipSuccess, "gemm_tiled: cannot raise the LDS limit: %s",                  \
                           hipGetErrorString(e));                                                          \
            raised = lds;                                                                                  \
        }                                                                                                  \
        gemm_direct_kernel<TN, TM, WN, WM, BK, NS, EPI, TC><<<grid, block, lds, stream>>>(                 \
            a, w, (TC*)C, M, N, k_len, lda, ldw, ldc, tiles_m, tiles_n, c_split_stride, link);             \
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
        for (int z = 0; z < splits; ++z) sum += *(const f32x4*)(ws + (int64_t)z * M * N + i);
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
                                hipStream_t stream, NormLink link = NormLink{}) {
    PICOLM_REQUIRE((!link.ssq && !link.next_w) || (N % 1024 == 0 && M <= link.rows && (link.rows == 16 || link.rows == 64)),
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
//   11: 128x128, 4 waves, four stages;
//   12: 128(n)x64(m), 4 waves, three stages;  13: 128(n)x32(m), 4 waves, four stages: for decode
//   batches of up to 64 or 32 rows, where the weights stream once and K may be split.
// Tiles staged through registers (any K that is a multiple of 8):
//   1: 128x128 (4 waves), 4: 256x256 (8 waves).
// The tile variant for a product by its shape.  Every variant moves about the same bytes a second
// from L2 into LDS, so the largest tile wins once its workgroups fill most of the 256 CUs.
// n_first > 0: the first n_first columns of 256x256 tiles go to variant 9 and the rest to variant
// 10: a last round that fills half of the CUs or less costs nearly a whole round, and the 256x128
// tile gives those columns twice the workgroups.
static int tiled_plan(int M, int N, int K, int& n_first) {
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
    return t256 >= 192 ? 9 : t128m >= 192 ? 10 : 11;
}

// Shares of a row's sum of squares that the tiled product of this shape leaves when it prepares a
// norm (one per column of tiles), or 0 if its kernel cannot take part in a split norm.
extern "C" int picolm_gemm_tiled_norm_parts(int M, int N, int K) {
    int n_first;
    const int variant = tiled_plan(M, N, K, n_first);
    return variant == 9 || variant == 10 ? ceil_div(N, 256) : variant == 11 ? ceil_div(N, 128) : 0;
}

static int gemm_tiled_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                             int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link);

extern "C" int picolm_gemm_tiled(const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                 int64_t lda, int64_t ldw, int64_t ldc, int epilogue, int variant,
                                 hipStream_t stream) {
    if (check_mfma_operands("gemm_tiled", A, W, M, N, K, lda, ldw, ldc, epilogue, c_dt)) return -1;
    if (M == 0) return 0;
    return gemm_tiled_linked(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, variant, stream, NormLink{});
}

static int gemm_tiled_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                             int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link) {
    if (variant == 0) {
        int n_first;
        variant = tiled_plan(M, N, K, n_first);
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
        PICOLM_REQUIRE(variant >= 9 && variant <= 11, "gemm_tiled: tile variant %d takes no part in a split norm", variant);
    switch (variant) {
        case 1: return launch_tiled<2, 2, 2, 2, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 4: return launch_tiled<2, 4, 4, 2, 1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 9: return launch_direct<2, 4, 4, 2, 64, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 10: return launch_direct<2, 2, 4, 2, 64, 3>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
        case 11: return launch_direct<2, 2, 2, 2, 64, 4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, 1, 0, link);
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
        case 9: rc = launch_direct<2, 4, 4, 2, 64, 2>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        case 10: rc = launch_direct<2, 2, 4, 2, 64, 3>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        case 11: rc = launch_direct<2, 2, 2, 2, 64, 4>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        case 12: rc = launch_direct<1, 2, 4, 1, 64, 3>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        case 13: rc = launch_direct<1, 1, 4, 1, 64, 4>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, stride); break;
        default: PICOLM_REQUIRE(false, "gemm_splitk: variant %d cannot split K", variant);
    }
    if (rc) return rc;
    return launch_splitk_reduce(ws, C, c_dt, M, N, ldc, splits, epilogue, stream);
}

// The products of a decode step with a norm split between them (see NormLink).  Up to 16 rows:
// `variant` as in picolm_gemm_skinny (0, 1, 7) or, with tiled != 0, tile variant 12 or 13; rows = 16.
// More than 64 rows (a prefill step): tiled, rows = a multiple of 64 of at least M, the tile
// variant by shape; either role, one share of the sums per column of tiles
// (picolm_gemm_tiled_norm_parts).
// 17 to 64 rows: tiled, variant 12, rows = 64; with splits > 1 (ws as in picolm_gemm_tiled_splitk)
// the kernel that adds the parts takes either role and N must be a multiple of 1024; uncut, the
// tile kernel can only take a prepared norm's statistics.
// next_*: this product (epilogue 1) prepares the norm that follows: next_h[M][ldc] and
// next_ssq[next_parts][rows], one row of partial sums per workgroup (ceil(N/16) of the skinny
// kernel, N/1024 of the adding kernel).  ssq, n_parts, norm_len, eps: this product's input rows
// are the next_h of a product that prepared their norm.
extern "C" int picolm_gemm_linked(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                  int64_t ldw, int64_t ldc, int epilogue, int tiled, int variant, int splits,
                                  float* ws, const float* next_w, void* next_h, float* next_ssq, int next_parts,
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
        return gemm_tiled_linked(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, 0, stream, link);
    }
    if (tiled && splits > 1) {
        PICOLM_REQUIRE(variant == 12 && ws != nullptr && ((uintptr_t)ws & 15) == 0 && N % 4 == 0,
                       "gemm_linked: a cut product needs tile variant 12, a workspace and N in multiples of 4");
        const int rc = launch_direct<1, 2, 4, 1, 64, 3>(A, W, ws, PICOLM_F32, M, N, K, lda, ldw, N, 0, stream, splits, (int64_t)M * N);
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
    if (variant == 0) variant = (M > 4 && N >= 16384 && K % SK_KSTEP == 0 && K <= 4 * 8 * SK_KSTEP && !next_w) ? 7 : 1;
    switch (variant) {
        case 1: return launch_skinny_sized<1>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, link);
        case 7: return launch_skinny_resident<4>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, link);
    }
    PICOLM_REQUIRE(false, "gemm_linked: skinny variant %d cannot take part in a split norm", variant);
}
