// Tile variants 14 and 15 of the kernel in gemm_direct.h: 192 and 320 columns by 256 rows, eight
// waves, two LDS stages, for products whose columns are a whole number of such tiles.
#include "gemm_direct.h"

int picolm_gemm_direct_wide_(int variant, const void* A, const void* W, void* C, int c_dt, int M, int N, int K,
                             int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t stream, int splits,
                             int64_t c_split_stride, NormLink link) {
    if (variant == 14)
        return launch_direct<3, 2, 2, 4, 64, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
    PICOLM_REQUIRE(variant == 15, "gemm_tiled: %d is no wide tile variant", variant);
    return launch_direct<5, 2, 2, 4, 64, 2>(A, W, C, c_dt, M, N, K, lda, ldw, ldc, epilogue, stream, splits, c_split_stride, link);
}
