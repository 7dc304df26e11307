// What the matrix-core product kernels share: vector types, the description of a norm split
// between two products, and the host helpers of their entry points.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include "common.h"
#include "api.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ bf16x8 load_chunk(const bf16_t* p) { return *(const bf16x8*)p; }
// a chunk of a matrix that this launch reads once: a non-temporal load (see stream_16_bytes_to_lds)
__device__ __forceinline__ bf16x8 stream_chunk(const bf16_t* p) { return __builtin_nontemporal_load((const bf16x8*)p); }
__device__ __forceinline__ bf16x8 zero_chunk() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
    return z;
}
// silu(g) * u with the hardware's 2^x and 1/x (an ulp each: far below the bfloat16 rounding of
// the products these kernels serve; the 32-bit path has its own formula in gemm_generic.hip).
// 2^x of a large x is inf and its reciprocal 0, so a very negative gate gives -0, as it should.
__device__ __forceinline__ float silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f)) * u;
}

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

static inline int check_mfma_operands(const char* who, const void* A, const void* W, int M, int N, int K, int64_t lda,
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

static inline int n_compute_units() {
    static int n_cus = 0;
    if (n_cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        n_cus = hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0
                    ? prop.multiProcessorCount : 256;
    }
    return n_cus;
}
// The entry points call each other's kernels across files through these.
// The skinny product for up to 16 rows with a split norm (variant 0, 1 or 7 as in picolm_gemm_skinny).
int picolm_gemm_skinny_linked_(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                               int64_t ldw, int64_t ldc, int epilogue, int variant, hipStream_t stream, NormLink link);
// The prefill's tile variants 9, 10, 11 (tiles straight into LDS), optionally cut along K.
int picolm_gemm_direct_prefill_(int variant, const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                                int64_t c_split_stride, NormLink link);
int picolm_gemm_direct_wide_(int variant, const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                             int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                             int64_t c_split_stride, NormLink link);
int picolm_gemm_direct_256x256_(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                                int64_t c_split_stride, NormLink link);
