// The prefill's tile variants 10 and 11 of the kernel in gemm_direct.h (variant 9 and the variants
// of 192 and 320 columns have files of their own), apart from the others so that they compile side
// by side.
#include "gemm_direct.h"

int picolm_gemm_direct_prefill_(int variant, const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                                int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                                int64_t c_split_stride, NormLink link) {
    switch (variant) {
        case 9: return picolm_gemm_direct_256x256_(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
        case 10: return launch_direct<2, 2, 4, 2, 64, 3>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
        case 14:
        case 15: return picolm_gemm_direct_wide_(variant, A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
        case 11: return launch_direct<2, 2, 2, 2, 64, 4, true>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
    }
    PICOLM_REQUIRE(false, "gemm_tiled: %d is no prefill tile variant", variant);
}
