// The error channel and device check of the library.
#include "common.h"
#include "api.h"
#include <stdarg.h>
#include <string.h>

static thread_local char g_error[512] = "";

void picolm_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* picolm_last_error(void) { return g_error; }

extern "C" int picolm_abi_version(void) { return 1; }

extern "C" int picolm_device_check(void) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    PICOLM_REQUIRE(e == hipSuccess, "no HIP device: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    PICOLM_REQUIRE(e == hipSuccess, "cannot query device %d: %s", dev, hipGetErrorString(e));
    PICOLM_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
                   "device %d is %s; these kernels are built for gfx950 only", dev, prop.gcnArchName);
    return 0;
}

// A read-only streaming kernel: what fraction of HBM's nominal bandwidth a plain sweep reaches
// on this machine.  The measurement harness quotes it next to the kernels' own figures.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, size_t n_vec,
                                                         unsigned* __restrict__ sink, int unroll4) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    unsigned acc = 0;
    if (unroll4) {
        for (; i + 3 * stride < n_vec; i += 4 * stride) {
            const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
            acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
        }
    }
    for (; i < n_vec; i += stride) {
        const uint4 a = src[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;      // keeps the loads alive; practically never true
}

extern "C" int picolm_read_probe(const void* src, size_t bytes, void* sink, int blocks, int unroll4,
                                 hipStream_t stream) {
    PICOLM_REQUIRE(bytes % 16 == 0 && blocks > 0, "read_probe: bytes must be a multiple of 16");
    read_probe_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const uint4*)src, bytes / 16, (unsigned*)sink, unroll4);
    PICOLM_LAUNCH_CHECK("read_probe");
    return 0;
}

// A compute-only kernel: what the matrix cores sustain on this machine with operands in
// registers (no memory traffic), for the measurement harness's "achievable" MFMA rate.
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;
// RANDOM: the operands are pseudo-random values of about the size of activations and weights, a
// different pair of registers for each of a wave's eight products (as in a tile product's wave:
// four operands one way, two the other).  With such operands the multipliers and adders switch as
// they do on real data, and the GPU's power limit, not the matrix cores' issue rate, sets the clock:
// this is the rate a real product can hope for.  With small integers (RANDOM = false) the same
// loop runs near the nominal peak.
template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_probe_kernel(float* __restrict__ sink, int iters) {
    probe_bf16x8 a[4], b[2];
    unsigned seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            seed = seed * 1664525u + 1013904223u;
            a[j][i] = RANDOM ? (__bf16)(((int)(seed >> 8) % 8192 - 4096) * (1.0f / 2048.0f)) : (__bf16)(float)(threadIdx.x % 7);
        }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            seed = seed * 1664525u + 1013904223u;
            b[j][i] = RANDOM ? (__bf16)(((int)(seed >> 8) % 8192 - 4096) * (0.02f / 2048.0f)) : (__bf16)(float)(threadIdx.x % 5);
        }
    probe_f32x16 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t % 4], b[t / 4], acc[t], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) s += acc[t][0];
    if (s == 12345.678f) sink[0] = s;
}

// flops done: blocks * 4 waves * iters * 8 * 32768
extern "C" int picolm_mfma_probe(void* sink, int blocks, int iters, int random_operands, hipStream_t stream) {
    PICOLM_REQUIRE(blocks > 0 && iters > 0, "mfma_probe: bad sizes");
    if (random_operands) mfma_probe_kernel<true><<<dim3(blocks), dim3(256), 0, stream>>>((float*)sink, iters);
    else mfma_probe_kernel<false><<<dim3(blocks), dim3(256), 0, stream>>>((float*)sink, iters);
    PICOLM_LAUNCH_CHECK("mfma_probe");
    return 0;
}
