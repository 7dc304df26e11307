// Token choice on the GPU.  Greedy: the first maximum of a row of logits
// (picolm/sampler.c:50-55, strict '>' keeps the lowest index among equals).
#include "common.h"
#include "api.h"

__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits,
                                                      int32_t* __restrict__ out, int V, int64_t ld) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (int64_t)blockIdx.x * ld;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) {   // first element seen, or strictly greater
            best = v;
            best_i = i;
        }
    }
    // a NaN never wins a '>' comparison; a row of NaNs yields its lowest index per thread
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(best_i, o, WAVE);
        if (oi != 0x7fffffff && (best_i == 0x7fffffff || ov > best || (ov == best && oi < best_i))) {
            best = ov;
            best_i = oi;
        }
    }
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (lane == 0) {
        sv[wave] = best;
        si[wave] = best_i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int n_waves = blockDim.x / WAVE;
        for (int w = 1; w < n_waves; ++w) {
            if (si[w] != 0x7fffffff && (best_i == 0x7fffffff || sv[w] > best || (sv[w] == best && si[w] < best_i))) {
                best = sv[w];
                best_i = si[w];
            }
        }
        out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
    }
}

extern "C" int picolm_argmax(const float* logits, int32_t* out, int n_rows, int V, int64_t ld,
                             hipStream_t stream) {
    PICOLM_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d ld=%lld", n_rows, V,
                   (long long)ld);
    if (n_rows == 0) return 0;
    argmax_kernel<<<dim3(n_rows), dim3(1024), 0, stream>>>(logits, out, V, ld);
    PICOLM_LAUNCH_CHECK("argmax");
    return 0;
}
