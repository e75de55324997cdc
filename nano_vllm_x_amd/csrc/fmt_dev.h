// Helpers of the kernels that take the activations' format as an argument (`fmt`: 0 bfloat16, 1 float16, 2 float32):
// element loads and stores through float, the dispatch of a launch on the format, and the description of a ragged step.
#pragma once
#include "nvx_dev.h"

namespace NVX_NS {

template <typename A> __device__ __forceinline__ float ld_f(const A* p, int64_t i) { return (float)p[i]; }
template <typename A> __device__ __forceinline__ void st_f(A* p, int64_t i, float v) { p[i] = (A)v; }

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

// sum over a workgroup of 256 threads; every thread gets the total.  `red` holds 4 floats; safe to call repeatedly.
__device__ __forceinline__ float block256_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// Where sequence b's tokens of this step are: first row, count, position of the first, state slot.
struct SeqSpan { int64_t q0; int64_t n; int64_t pos0; int slot; };
__device__ __forceinline__ SeqSpan seq_span(int b, const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot) {
    SeqSpan s;
    s.q0 = qo_indptr ? qo_indptr[b] : b;
    s.n = qo_indptr ? qo_indptr[b + 1] - s.q0 : 1;
    s.pos0 = pos0[b];
    s.slot = state_slot[b];
    return s;
}

}  // namespace NVX_NS

#define NVX_FMT_CALL(fmt, CALL)                                             \
    do {                                                                    \
        if ((fmt) == 0) { typedef __bf16 A_; CALL; }                        \
        else if ((fmt) == 1) { typedef _Float16 A_; CALL; }                 \
        else { typedef float A_; CALL; }                                    \
    } while (0)
