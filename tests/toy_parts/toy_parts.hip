// Two toy parts with kernels of their own, for the tests: what a part outside the library needs
// in order to run inside the engine's step (csrc/engine.h, PICOLM_OP_CALL).  Each is a C function
// that the engine hands the running step to, and a kernel that it queues on the step's stream.
// Nothing here is part of the library; it is built into a library of its own beside this file.
//
//   toy_running_mean   a mixer that keeps, per sequence, the sum of its inputs and their count:
//                      out[t] += W mean(in[0..t]); state per slot: D sums and the count, float
//   toy_centered_norm  out = (x - mean(x)) / sqrt(var(x) + eps) * w + b, on every row or on the
//                      wanted rows, in float or bfloat16
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "engine.h"

extern "C" void picolm_set_error_message(const char* message);

struct toy_running_mean_args {
    const float* w;      // [D][D], row-major: out = W mean
    int32_t D;
    int32_t in_bf16;     // the input rows are bfloat16 (else float)
};

struct toy_centered_norm_args {
    const float* w;
    const float* b;
    int32_t D;
    float eps;
    int32_t out_bf16;
};

// bfloat16 is the upper half of a float; rounding to it is to nearest, ties to even
__device__ static float bf16_to_float(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ static uint16_t float_to_bf16(float f) {
    const uint32_t u = __float_as_uint(f);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
__device__ static float load_in(const void* p, size_t i, int bf16) {
    return bf16 ? bf16_to_float(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}

// One workgroup per sequence walks its rows in order; thread c owns column c of the sums (in LDS)
// and output column c.
__global__ void toy_running_mean_kernel(const void* in, int in_stride, int in_bf16, float* out, int out_stride, float* state,
                                        int state_stride, const float* w, int D, const int32_t* seq_slot,
                                        const int32_t* cu_seqlens) {
    extern __shared__ float mean[];
    const int seq = blockIdx.x;
    float* st = state + (size_t)seq_slot[seq] * state_stride;
    const int row0 = cu_seqlens[seq], row1 = cu_seqlens[seq + 1];
    float count = st[D];
    for (int row = row0; row < row1; ++row) {
        count += 1.f;
        for (int c = threadIdx.x; c < D; c += blockDim.x) {
            const float s = st[c] + load_in(in, (size_t)row * in_stride + c, in_bf16);
            st[c] = s;
            mean[c] = s / count;
        }
        __syncthreads();
        for (int c = threadIdx.x; c < D; c += blockDim.x) {
            float acc = 0.f;
            for (int k = 0; k < D; ++k) acc += mean[k] * w[(size_t)c * D + k];
            out[(size_t)row * out_stride + c] += acc;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) st[D] = count;
}

extern "C" int toy_running_mean(void* user, const picolm_step_view* v) {
    const toy_running_mean_args* a = (const toy_running_mean_args*)user;
    if (v->struct_bytes != (int32_t)sizeof(picolm_step_view) || !v->state || !v->in || !v->out ||
        v->state_bytes_per_slot != (int64_t)(a->D + 1) * 4) {
        picolm_set_error_message("toy_running_mean: the step view does not fit (buffers, or state of D + 1 floats a slot)");
        return -1;
    }
    const int in_size = a->in_bf16 ? 2 : 4;
    toy_running_mean_kernel<<<v->n_seq, 64, a->D * sizeof(float), v->stream>>>(
        v->in, v->in_row_bytes / in_size, a->in_bf16, (float*)v->out, v->out_row_bytes / 4, (float*)v->state, a->D + 1, a->w, a->D,
        v->seq_slot, v->cu_seqlens);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// One workgroup of 64 lanes per output row.
__global__ void toy_centered_norm_kernel(const float* x, int x_stride, void* out, int out_stride, int out_bf16, const float* w,
                                         const float* b, int D, float eps, const int32_t* rows) {
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * x_stride;
    float s = 0.f;
    for (int c = threadIdx.x; c < D; c += 64) s += xr[c];
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    const float mean = s / D;
    float q = 0.f;
    for (int c = threadIdx.x; c < D; c += 64) q += (xr[c] - mean) * (xr[c] - mean);
    for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o);
    const float r_std = 1.f / sqrtf(q / D + eps);
    for (int c = threadIdx.x; c < D; c += 64) {
        const float y = (xr[c] - mean) * r_std * w[c] + b[c];
        if (out_bf16) ((uint16_t*)out)[(size_t)r * out_stride + c] = float_to_bf16(y);
        else ((float*)out)[(size_t)r * out_stride + c] = y;
    }
}

extern "C" int toy_centered_norm(void* user, const picolm_step_view* v) {
    const toy_centered_norm_args* a = (const toy_centered_norm_args*)user;
    if (v->struct_bytes != (int32_t)sizeof(picolm_step_view) || !v->in || !v->out) {
        picolm_set_error_message("toy_centered_norm: the step view does not fit");
        return -1;
    }
    if (v->rows == 0) return 0;
    // over the wanted rows it gathers them, unless they are the step's rows in order
    const int32_t* rows = v->rows == v->n_tokens && (v->rows != v->n_wanted || v->every_row_wanted) ? nullptr : v->want_rows;
    toy_centered_norm_kernel<<<v->rows, 64, 0, v->stream>>>((const float*)v->in, v->in_row_bytes / 4, v->out,
                                                             v->out_row_bytes / (a->out_bf16 ? 2 : 4), a->out_bf16, a->w, a->b, a->D,
                                                             a->eps, rows);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
