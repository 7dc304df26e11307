// Shared device helpers for the gfx950 kernels: storage types, conversions, reductions,
// and the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

// ---- element types ------------------------------------------------------------------
// Tensors are float (32-bit) or bf16 stored as uint16_t.  All arithmetic is float.
#ifndef PICOLM_ELEMENT_TYPES
#define PICOLM_ELEMENT_TYPES
enum { PICOLM_F32 = 0, PICOLM_BF16 = 1 };
#endif
typedef uint16_t bf16_t;

#define PAGE_TOKENS 64       // tokens of one cache page; also the key tile of attention
#define WAVE 64

__device__ __forceinline__ float bf16_bits_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}
// Round to nearest, ties to even; NaN stays NaN.  (The conversion is one instruction on gfx950.)
__device__ __forceinline__ bf16_t f32_to_bf16_bits(float f) {
    return __builtin_bit_cast(bf16_t, (__bf16)f);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_bits_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16_bits(v); }

// ---- loads from global memory straight into LDS ------------------------------------------
// global_load_lds_dwordx4: the 64 lanes of a wave bring 16 bytes each to 1 KB of LDS in a row, with
// no staging registers and no LDS store instructions.  Inline assembly, so that a wait for "all
// but the newest loads" (s_waitcnt vmcnt(n)) stays as written: the compiler, when it knows of such
// loads, waits for all of them before any LDS read.  M0 carries the LDS address of the wave's 1 KB.
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
// The same for bytes that are read once (weights of a product with one row of tiles): marked
// non-temporal, they pass the caches without displacing what is read again.  A sweep over 4 GB
// reaches 7.0 to 7.2 TB/s with such loads and 6.2 without.
__device__ __forceinline__ void stream_16_bytes_to_lds(unsigned byte_offset, const void* base, unsigned lds_address) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :
                 : "v"(byte_offset), "s"(base), "s"(lds_address)
                 : "memory");
}
template <int N_OUTSTANDING>
__device__ __forceinline__ void wait_for_loads() {      // vmcnt(N), other counters untouched
    static_assert(N_OUTSTANDING < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt((N_OUTSTANDING & 15) | (7 << 4) | (15 << 8) | ((N_OUTSTANDING >> 4) << 14));
}


// ---- reductions ---------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
// Sum over a block of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < n_waves; ++i) t += scratch[i];
    return t;
}

// ---- host side ------------------------------------------------------------------------
// Every entry point returns 0 or a negative code and leaves a message for
// picolm_last_error().
void picolm_set_error(const char* fmt, ...);

#define PICOLM_REQUIRE(cond, ...)                         \
    do {                                                  \
        if (!(cond)) {                                    \
            picolm_set_error(__VA_ARGS__);                \
            return -1;                                    \
        }                                                 \
    } while (0)

#define PICOLM_LAUNCH_CHECK(name)                                                     \
    do {                                                                              \
        hipError_t e__ = hipGetLastError();                                           \
        if (e__ != hipSuccess) {                                                      \
            picolm_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));  \
            return -2;                                                                \
        }                                                                             \
    } while (0)

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
