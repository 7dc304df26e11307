// The product a layer asks for, C = A W^T with its epilogue: which kernel runs for which operand
// types and sizes, and how an RMSNorm between two products is shared by them.  Host code only;
// the engine's step and the Python face of the library both call picolm_linear, so the choice is
// made in one place.  picolm picks its matmul by the weight's type alone (picolm/tensor.c:2174,
// picolm/quant.c:4957-4968); here the number of rows decides as well:
//   not bf16 x bf16, or K no multiple of 8      the float kernel on the vector ALU
//   up to 16 rows                               skinny: weights streamed once into MFMA operands
//                                               (tiles of 128 weight rows through LDS where there
//                                               are 128 such tiles and more)
//   17 to 64 rows                               128-row weight tiles through LDS, cut along K
//                                               when there are fewer tiles than CUs
//   more than 64 rows                           the prefill's tile variants by shape
#include "common.h"
#include "api.h"
#include "gemm_mfma.h"

#define PICOLM_SPLITK_WS_FLOATS (8 << 20)      // 32 MB of partial sums: splits * M * N may not exceed it

extern "C" int64_t picolm_linear_workspace_floats(void) { return PICOLM_SPLITK_WS_FLOATS; }

static bool mfma_takes(const void* a, int a_dt, const void* w, int w_dt, int c_dt, int K, int epilogue) {
    if (a_dt != PICOLM_BF16 || w_dt != PICOLM_BF16) return false;
    if (K % 8 != 0 || ((uintptr_t)a & 15) || ((uintptr_t)w & 15)) return false;
    if (epilogue == 1) return c_dt == PICOLM_F32;
    return true;
}

// The tile variant for a decode batch of 17 to 64 rows: tiles of 128 weight rows by 64 activation
// rows, or by 32 where that is enough (measured 5 to 9 % faster there).
static int medium_variant(int M) { return M <= 32 ? 13 : 12; }

// Into how many parts along K a product of 17..64 rows is cut: its tiles hold 128 weight rows
// each, and every CU should have one; never a few more workgroups than CUs, whose last ones run
// while most CUs wait (measured with weights from memory at 32 rows: 80 tiles, 10,240 x 8,192,
// cut in two 36.7 us and in four 43.0; 40 tiles, 5,120 x 13,824, in four 33.6 and in eight 37.8;
// 160 tiles, 20,480 x 4,096, uncut 31.6 and in two 41.7).
extern "C" int picolm_linear_medium_splits(int M, int N, int K);
static int medium_splits(int M, int N, int K) { return picolm_linear_medium_splits(M, N, K); }
extern "C" int picolm_linear_medium_splits(int M, int N, int K) {
    const int tiles = (N + 127) / 128;
    if (tiles >= 200 || N % 4) return 1;
    int s = 8;
    while (s > 1 && (tiles * s > n_compute_units() || K % (64 * s) || (int64_t)s * M * N > PICOLM_SPLITK_WS_FLOATS)) s /= 2;
    return s;
}

// Rows that the partial sums of a split norm are kept for in a step of M rows: 16 or 64 in a
// decode step, every row (in whole 64s) otherwise.
extern "C" int picolm_linear_norm_rows(int M) { return M <= 16 ? 16 : M <= 64 ? 64 : (M + 63) / 64 * 64; }

// Partial sums per row that a product of M rows, N output columns and K input columns leaves for
// the norm that follows: one per workgroup (or column of tiles) of the kernel that finishes the
// rows.  0: that kernel cannot.
extern "C" int picolm_linear_norm_parts(int M, int N, int K) {
    if (M <= 16) return (N + 15) / 16;
    if (M <= 64) return N / 1024;
    return picolm_gemm_tiled_norm_parts(M, N, K, PICOLM_SPLITK_WS_FLOATS);
}

// Whether the product for these operands can take part in a norm split between two products:
// prepare the next one (with the accumulating epilogue), or else take a prepared one's statistics.
// Up to 16 rows every matrix-core product can do both.  For 17 to 64 rows the kernel that adds the
// parts of a product cut along K does either for N in multiples of 1024, and the tile kernel of an
// uncut product can take the statistics.  Above that the tile kernels whose tiles go straight
// into LDS (K in multiples of 64) do both.
extern "C" int picolm_linear_links_norms(const void* a, int a_dt, const void* w, int w_dt, int c_dt, int M, int N,
                                         int K, int epilogue, int prepares) {
    if (!mfma_takes(a, a_dt, w, w_dt, c_dt, K, epilogue)) return 0;
    if (M <= 16) return 1;
    if (K % 64) return 0;
    if (M > 64) return picolm_linear_norm_parts(M, N, K) > 0;
    const bool cut = medium_splits(M, N, K) > 1;
    return prepares ? (cut && N % 1024 == 0) : (!cut || N % 1024 == 0);
}

// C (=, +=, = silu-gated) A W^T for row-major A[M][K], W[N][K], C[M][N or N/2], all contiguous.
// next_w, next_h, next_ssq, next_parts: with the accumulating epilogue, also leave
//   next_h[M][N] = bf16(C * next_w) and next_ssq[next_parts][rows] partial sums of C^2
//   (rows = picolm_linear_norm_rows(M), next_parts = picolm_linear_norm_parts(M, N, K)).
// ssq, n_parts, norm_len, eps: A is such a next_h; the sums are multiplied by
//   1 / sqrt(sum(x^2) / norm_len + eps).
// Either role needs picolm_linear_links_norms to say yes.  ws: picolm_linear_workspace_floats()
// floats for the partial sums of products cut along K (one buffer a stream: kernels of a stream
// run in order); it may be null, then no product is cut.
extern "C" int picolm_linear(const void* A, int a_dt, const void* W, int w_dt, void* C, int c_dt, int M, int N, int K,
                             int epilogue, const float* next_w, void* next_h, float* next_ssq, int next_parts,
                             const float* ssq, int n_parts, int norm_len, float eps, float* ws, hipStream_t stream) {
    PICOLM_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
    PICOLM_REQUIRE(epilogue >= 0 && epilogue <= 2, "linear: unknown epilogue %d", epilogue);
    const int64_t ldc = epilogue == 2 ? N / 2 : N;
    const bool linked = next_w != nullptr || ssq != nullptr;
    if (!mfma_takes(A, a_dt, W, w_dt, c_dt, K, epilogue)) {
        PICOLM_REQUIRE(!linked, "linear: these operands cannot share a norm with another product");
        return picolm_gemm_generic(A, a_dt, W, w_dt, C, c_dt, M, N, K, K, K, ldc, epilogue, stream);
    }
    if (next_w) {
        PICOLM_REQUIRE(epilogue == 1, "linear: only the accumulating epilogue prepares a norm");
        PICOLM_REQUIRE(picolm_linear_links_norms(A, a_dt, W, w_dt, c_dt, M, N, K, epilogue, 1),
                       "linear: a product of %d x %d x %d cannot prepare a norm", M, N, K);
        PICOLM_REQUIRE(next_h && next_ssq && next_parts == picolm_linear_norm_parts(M, N, K),
                       "linear: the buffers for the next norm do not fit the product");
    }
    if (ssq) {
        PICOLM_REQUIRE(picolm_linear_links_norms(A, a_dt, W, w_dt, c_dt, M, N, K, epilogue, 0),
                       "linear: a product of %d x %d x %d cannot take a prepared norm", M, N, K);
        PICOLM_REQUIRE(norm_len == K && n_parts > 0, "linear: the statistics are not those of this product's input rows");
    }
    const int rows = picolm_linear_norm_rows(M);
    const int64_t ws_floats = ws ? PICOLM_SPLITK_WS_FLOATS : 0;
    if (M > 64)         // the tile variant by shape, cut along K where it has few tiles
        return picolm_gemm_linked(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, 1, 0, 1, ws, ws_floats, next_w, next_h,
                                  next_ssq, next_parts, ssq, n_parts, norm_len, eps, rows, stream);
    if (M > 16 && (linked || K % 64 == 0)) {
        // a decode batch too wide to re-read its activations for every 16 weight rows: tiles of 128
        // weight rows through LDS, cut along K where there are few of them
        const int variant = medium_variant(M);
        const int splits = ws ? medium_splits(M, N, K) : 1;
        if (!linked) return picolm_gemm_tiled_splitk(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, variant, splits, ws, stream);
        return picolm_gemm_linked(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, 1, variant, splits, splits > 1 ? ws : nullptr,
                                  ws_floats, next_w, next_h, next_ssq, next_parts, ssq, n_parts, norm_len, eps, rows, stream);
    }
    // enough weight rows for half a round and more of 128-row tiles: the tile kernel, whose loads
    // cover whole lines, streams the weights past the caches (measured with weights from memory,
    // 28,672 x 4,096: 37.0 us against the skinny kernel's 40.2 at one row, 37.2 against 43.7 at
    // eight; 57,344 x 8,192: 142 against 164 and 144 against 177; 12,288 rows, 96 tiles, are
    // better off skinny: 19 against 26 us).  Up to eight rows of many rounds (a vocabulary) stay
    // skinny, two staged workgroups a CU: 155 against 167 us for 128,256 rows at one row, 154
    // against 172 at eight; and so do up to eight rows of a product whose tiles reach little more
    // than half of the CUs, unless K is long (16,384 x 2,048: 14.3 against 16.3 us at one row, 14.7
    // against 16.9 at eight; x 4,096: 23.5 against 26.7 and 22.3 against 27.9; 18,432 x 4,096: 24.9
    // against 27.7 and 24.4 against 28.4; 19,456 x 4,096: 27.0 against 27.6 and 26.1 against 28.9;
    // 16,384 x 8,192: 48.6 against 47.2 and 52.1 against 48.8).
    const bool one_round = M <= 16 && K % 64 == 0 && N >= 16384 &&
                           (M > 8 || (N <= 512 * 128 && (N > 72 * n_compute_units() || K > 4096)));
    if (!linked) {
        if (one_round) return picolm_gemm_tiled_splitk(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, 13, 1, nullptr, stream);
        return picolm_gemm_skinny(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, 0, stream);
    }
    const int tiled = one_round && !next_w;
    return picolm_gemm_linked(A, W, C, c_dt, M, N, K, K, K, ldc, epilogue, tiled, tiled ? 13 : 0, 1, nullptr, ws_floats,
                              next_w, next_h, next_ssq, next_parts, ssq, n_parts, norm_len, eps, rows, stream);
}
