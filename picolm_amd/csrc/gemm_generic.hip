// C[M,N] = A[M,K] * W[N,K]^T with float accumulation on the vector ALU, any sizes and any
// mix of float / bf16 operands.  This is the product of the true 32-bit path (no matrix
// cores, no reduced precision anywhere) and the fallback for shapes the MFMA kernels refuse.
// picolm computes the same product row by row: out[d] = dot(W[d,:], x) (picolm/tensor.c:839,
// :2174; float accumulate picolm/quant.c:4957-4968).
#include "common.h"
#include "api.h"

#define GG_BM 64
#define GG_BN 64
#define GG_BK 16
#define GG_PAD 4

// epilogue: 0 store, 1 C += acc (C is float), 2 C[m][n/2] = silu(acc[n]) * acc[n+1] for even n
template <typename TA, typename TW, typename TC, int EPI>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A,
                                                           const TW* __restrict__ W,
                                                           TC* __restrict__ C, int M, int N, int K,
                                                           int64_t lda, int64_t ldw, int64_t ldc) {
    __shared__ float As[GG_BK][GG_BM + GG_PAD];
    __shared__ float Ws[GG_BK][GG_BN + GG_PAD];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * GG_BM, n0 = blockIdx.x * GG_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GG_BK) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int idx = tid + it * 256;
            const int r = idx / GG_BK, c = idx % GG_BK;
            const int k = k0 + c;
            const int m = m0 + r, n = n0 + r;
            As[c][r] = (m < M && k < K) ? to_f32<TA>(A[(int64_t)m * lda + k]) : 0.f;
            Ws[c][r] = (n < N && k < K) ? to_f32<TW>(W[(int64_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GG_BK; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        if (EPI == 2) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const int n = n0 + tx * 4 + j;
                if (n + 1 < N) {
                    const float g = acc[i][j], u = acc[i][j + 1];
                    C[(int64_t)m * ldc + n / 2] = from_f32<TC>(g / (1.0f + expf(-g)) * u);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n >= N) continue;
                TC* p = C + (int64_t)m * ldc + n;
                if (EPI == 1)
                    *p = from_f32<TC>(to_f32<TC>(*p) + acc[i][j]);
                else
                    *p = from_f32<TC>(acc[i][j]);
            }
        }
    }
}

template <typename TA, typename TW, typename TC>
static int launch_generic(const void* A, const void* W, void* C, int M, int N, int K, int64_t lda,
                          int64_t ldw, int64_t ldc, int epi, hipStream_t stream) {
    dim3 grid(ceil_div(N, GG_BN), ceil_div(M, GG_BM)), block(256);
    const TA* a = (const TA*)A;
    const TW* w = (const TW*)W;
    TC* c = (TC*)C;
    if (epi == 0)
        gemm_generic_kernel<TA, TW, TC, 0><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc);
    else if (epi == 1)
        gemm_generic_kernel<TA, TW, TC, 1><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc);
    else
        gemm_generic_kernel<TA, TW, TC, 2><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc);
    PICOLM_LAUNCH_CHECK("gemm_generic");
    return 0;
}

extern "C" int picolm_gemm_generic(const void* A, int a_dt, const void* W, int w_dt, void* C,
                                   int c_dt, int M, int N, int K, int64_t lda, int64_t ldw,
                                   int64_t ldc, int epilogue, hipStream_t stream) {
    PICOLM_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    PICOLM_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm: unknown epilogue %d", epilogue);
    PICOLM_REQUIRE(epilogue != 1 || c_dt == PICOLM_F32, "gemm: accumulation needs a float output");
    PICOLM_REQUIRE(epilogue != 2 || N % 2 == 0, "gemm: the gated epilogue needs an even N, got %d", N);
    PICOLM_REQUIRE(lda >= K && ldw >= K && ldc >= (epilogue == 2 ? N / 2 : N),
                   "gemm: leading dimensions too small (lda=%lld ldw=%lld ldc=%lld)", (long long)lda,
                   (long long)ldw, (long long)ldc);
    PICOLM_REQUIRE(ceil_div(M, GG_BM) <= 65535, "gemm: M=%d needs more than 65535 row tiles", M);
    if (M == 0) return 0;
    const int key = a_dt * 4 + w_dt * 2 + c_dt;
    switch (key) {
        case 0: return launch_generic<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 1: return launch_generic<float, float, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 2: return launch_generic<float, bf16_t, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 3: return launch_generic<float, bf16_t, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 4: return launch_generic<bf16_t, float, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 5: return launch_generic<bf16_t, float, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 6: return launch_generic<bf16_t, bf16_t, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
        case 7: return launch_generic<bf16_t, bf16_t, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, stream);
    }
    PICOLM_REQUIRE(false, "gemm: unknown dtypes a=%d w=%d c=%d", a_dt, w_dt, c_dt);
}
