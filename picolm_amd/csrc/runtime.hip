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

extern "C" void picolm_set_error_message(const char* message) { picolm_set_error("%s", message ? message : ""); }

extern "C" int picolm_abi_version(void) { return 2; }

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

// A read-only streaming kernel: what fraction of HBM's nominal bandwidth a sweep reaches on this
// machine.  The measurement harness quotes it next to the kernels' own figures.  Each workgroup
// sweeps a contiguous share, 4 KB at a time with eight loads of a thread in flight; with
// `streaming` the loads are non-temporal, as the kernels' loads of weights and cached keys and
// values are that a launch reads once (4 GB: 7.0 to 7.2 TB/s against 6.2 with plain loads).
typedef __attribute__((ext_vector_type(4))) unsigned probe_u4;
template <bool STREAMING>
__global__ __launch_bounds__(256) void read_probe_kernel(const probe_u4* __restrict__ src, size_t n_vec,
                                                         unsigned* __restrict__ sink) {
    const size_t per = n_vec / gridDim.x / 2048 * 2048;      // whole rounds of eight loads a thread; the rest is not read
    const probe_u4* p = src + per * blockIdx.x + threadIdx.x;
    unsigned acc = 0;
    for (size_t i = 0; i < per; i += 2048) {
        probe_u4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = STREAMING ? __builtin_nontemporal_load(p + i + u * 256) : p[i + u * 256];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;      // keeps the loads alive; practically never true
}

// Returns in *bytes_read (if given) what the launch reads: whole rounds of 32 KB a workgroup.
extern "C" int picolm_read_probe(const void* src, size_t bytes, void* sink, int blocks, int streaming,
                                 hipStream_t stream) {
    PICOLM_REQUIRE(bytes % 16 == 0 && blocks > 0 && bytes / 16 / blocks >= 2048,
                   "read_probe: bytes must be a multiple of 16 and at least 32 KB a workgroup");
    if (streaming) read_probe_kernel<true><<<dim3(blocks), dim3(256), 0, stream>>>((const probe_u4*)src, bytes / 16, (unsigned*)sink);
    else read_probe_kernel<false><<<dim3(blocks), dim3(256), 0, stream>>>((const probe_u4*)src, bytes / 16, (unsigned*)sink);
    PICOLM_LAUNCH_CHECK("read_probe");
    return 0;
}
extern "C" size_t picolm_read_probe_bytes(size_t bytes, int blocks) {
    return blocks > 0 ? bytes / 16 / blocks / 2048 * 2048 * (size_t)blocks * 16 : 0;
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
