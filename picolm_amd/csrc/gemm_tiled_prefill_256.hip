// Tile variant 9 of the kernel in gemm_direct.h: 256x256 tiles, eight waves, two LDS stages.
#include "gemm_direct.h"

int picolm_gemm_direct_256x256_(const void* A, const void* W, void* C, int c_dt, int M, int N, int K, int64_t lda,
                                int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                                int64_t c_split_stride, NormLink link) {
    return launch_direct<2, 4, 4, 2, 64, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
}
