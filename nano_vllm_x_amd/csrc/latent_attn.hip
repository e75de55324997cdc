// Latent attention: every token caches ONE vector c (kv_rank values); a head's keys and values are linear maps of it.
// The maps are folded into the query and the output, so the kernel attends over the cached latents themselves:
//     score_j = scale * q~ . c_j   (q~ = the head's key map transposed, applied to its query),   o~ = sum_j p_j c_j
// and the head's output is its value map applied to o~.  All heads of a token share the same keys, and a key row
// serves as the value row too.  Scores, softmax weights and the weighted sum are float32; the cache holds the
// activations' format (`fmt`: 0 bfloat16, 1 float16, 2 float32).  No positions enter.
#include "nvx_dev.h"

namespace NVX_NS {

template <typename A> __device__ __forceinline__ float la_ld(const A* p, int64_t i) { return (float)p[i]; }
template <typename A> __device__ __forceinline__ void la_st(A* p, int64_t i, float v) { p[i] = (A)v; }

__device__ __forceinline__ float la_block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ---- what follows the down projections --------------------------------------------------------------------------------
// x[t] = [ query latent (q_rank) | key/value latent (kv_rank) | one output-gate pre-activation per head ].
//   cq[t]           = query latent / rms * w_q                     (activation format, feeds the query up-projection)
//   cache[slot[t]]  = key/value latent / rms * w_kv                (a negative slot: not stored)
//   gate[t][h]      = sigmoid(pre-activation)                      (float32)
template <typename A>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const A* __restrict__ x, int64_t x_stride, const float* __restrict__ w_q, const float* __restrict__ w_kv, float eps,
    const int64_t* __restrict__ slots, A* __restrict__ cq, A* __restrict__ cache, int64_t n_slots, float* __restrict__ gate,
    int q_rank, int kv_rank, int heads) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* r = x + t * x_stride;
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += 256) { const float v = la_ld(r, c); ss += v * v; }
    const float rq = 1.0f / sqrtf(la_block_sum(ss, red) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += 256) la_st(cq, t * q_rank + c, la_ld(r, c) * rq * w_q[c]);
    ss = 0.f;
    for (int c = threadIdx.x; c < kv_rank; c += 256) { const float v = la_ld(r, q_rank + c); ss += v * v; }
    const float rk = 1.0f / sqrtf(la_block_sum(ss, red) / (float)kv_rank + eps);
    const int64_t slot = slots[t];
    if (slot >= 0 && slot < n_slots)
        for (int c = threadIdx.x; c < kv_rank; c += 256) la_st(cache, slot * kv_rank + c, la_ld(r, q_rank + c) * rk * w_kv[c]);
    for (int h = threadIdx.x; h < heads; h += 256)
        gate[t * heads + h] = 1.0f / (1.0f + expf(-la_ld(r, q_rank + kv_rank + h)));
}

// ---- attention over the cached latents ------------------------------------------------------------------------------
// One workgroup per (query token, group of HG heads).  Keys come in tiles of 256: first every thread scores one key
// against the group's folded queries (held in LDS), the tile's weights go to LDS, then every thread owns output
// columns and adds the tile's weighted rows.  Running maximum and sum per head (online softmax).
// q / out: (heads, tokens, rank).  Token t of sequence b sees the sequence's keys 0 .. kv_len[b] - q_len[b] + local(t).
// kv_indices + kv_start[b]: the slots of sequence b's tokens in order (a flat list with offsets, or rows of a table).
#define LA_KT 256
#define LA_MAXC 4      // output columns per thread: rank <= 256 * LA_MAXC

template <typename A, int HG>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const A* __restrict__ q, const A* __restrict__ cache, const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ tok_seq,
    const float* __restrict__ gate, A* __restrict__ out, int heads, int rank, int64_t n_tok, float scale) {
    extern __shared__ float lds[];
    float* q_l = lds;                          // HG * rank
    float* p_l = q_l + HG * rank;              // LA_KT * HG
    int* slot_l = (int*)(p_l + LA_KT * HG);    // LA_KT
    float* red = (float*)(slot_l + LA_KT);     // 4 * HG
    const int64_t t = blockIdx.x;
    const int h0 = blockIdx.y * HG;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : t;
    const int64_t q_len = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    const int64_t n_keys = (int64_t)kv_len[b] - q_len + (t - q0) + 1;
    const int32_t* idx = kv_indices + kv_start[b];
    for (int i = tid; i < HG * rank; i += 256) {
        const int h = h0 + i / rank;
        q_l[i] = h < heads ? la_ld(q, ((int64_t)h * n_tok + t) * rank + (i % rank)) : 0.f;
    }
    float m_run[HG], l_run[HG], acc[LA_MAXC][HG];
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        m_run[h] = -INFINITY;
        l_run[h] = 0.f;
#pragma unroll
        for (int k = 0; k < LA_MAXC; ++k) acc[k][h] = 0.f;
    }
    for (int64_t k0 = 0; k0 < n_keys; k0 += LA_KT) {
        const int64_t j = k0 + tid;
        const bool valid = j < n_keys;
        const int slot = valid ? idx[j] : 0;
        __syncthreads();                                   // q_l is written; the previous tile's p_l and slot_l are read
        slot_l[tid] = slot;
        float s[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) s[h] = 0.f;
        if (valid) {
            const A* row = cache + (int64_t)slot * rank;
            for (int r = 0; r < rank; ++r) {
                const float c = la_ld(row, r);
#pragma unroll
                for (int h = 0; h < HG; ++h) s[h] += q_l[h * rank + r] * c;
            }
        }
        // tile maximum per head
        float alpha[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            s[h] = valid ? s[h] * scale : -INFINITY;
            const float wm = wave_max(s[h]);
            if (lane == 0) red[wv * HG + h] = wm;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const float tm = fmaxf(fmaxf(red[h], red[HG + h]), fmaxf(red[2 * HG + h], red[3 * HG + h]));
            const float m_new = fmaxf(m_run[h], tm);       // finite: every tile has at least one visible key
            alpha[h] = expf(m_run[h] - m_new);              // first tile: exp(-inf) = 0
            m_run[h] = m_new;
            s[h] = valid ? expf(s[h] - m_new) : 0.f;
            p_l[tid * HG + h] = s[h];
        }
        __syncthreads();                                   // p_l and slot_l are complete; red has been read
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const float ws = wave_sum(s[h]);
            if (lane == 0) red[wv * HG + h] = ws;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            l_run[h] = l_run[h] * alpha[h] + (red[h] + red[HG + h] + red[2 * HG + h] + red[3 * HG + h]);
#pragma unroll
            for (int k = 0; k < LA_MAXC; ++k) acc[k][h] *= alpha[h];
        }
        const int n_here = (int)((n_keys - k0) < LA_KT ? (n_keys - k0) : LA_KT);
        for (int jj = 0; jj < n_here; ++jj) {
            const A* row = cache + (int64_t)slot_l[jj] * rank;
#pragma unroll
            for (int k = 0; k < LA_MAXC; ++k) {
                const int c = tid + k * 256;
                if (c < rank) {
                    const float v = la_ld(row, c);
#pragma unroll
                    for (int h = 0; h < HG; ++h) acc[k][h] += p_l[jj * HG + h] * v;
                }
            }
        }
    }
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        if (h0 + h >= heads) continue;
        const float f = (gate ? gate[t * heads + h0 + h] : 1.0f) / l_run[h];
#pragma unroll
        for (int k = 0; k < LA_MAXC; ++k) {
            const int c = tid + k * 256;
            if (c < rank) la_st(out, ((int64_t)(h0 + h) * n_tok + t) * rank + c, acc[k][h] * f);
        }
    }
}

template <typename A>
static void launch_prep(const void* x, int64_t x_stride, const float* w_q, const float* w_kv, float eps, const int64_t* slots, void* cq,
                        void* cache, int64_t n_slots, float* gate, int64_t n_tok, int q_rank, int kv_rank, int heads, hipStream_t s) {
    hipLaunchKernelGGL(latent_prep_kernel<A>, dim3((unsigned)n_tok), dim3(256), 0, s, (const A*)x, x_stride, w_q, w_kv, eps, slots, (A*)cq,
                       (A*)cache, n_slots, gate, q_rank, kv_rank, heads);
}

template <typename A>
static void launch_attn(const void* q, const void* cache, const int32_t* kv_indices, const int64_t* kv_start, const int32_t* kv_len,
                        const int32_t* qo_indptr, const int32_t* tok_seq, const float* gate, void* out, int heads, int rank, int64_t n_tok,
                        float scale, hipStream_t s) {
    constexpr int HG = 4;
    const size_t lds = (size_t)(HG * rank + LA_KT * HG + LA_KT + 4 * HG) * 4;
    hipLaunchKernelGGL((latent_attn_kernel<A, HG>), dim3((unsigned)n_tok, (unsigned)((heads + HG - 1) / HG)), dim3(256), lds, s,
                       (const A*)q, (const A*)cache, kv_indices, kv_start, kv_len, qo_indptr, tok_seq, gate, (A*)out, heads, rank, n_tok,
                       scale);
}

}  // namespace NVX_NS

using namespace NVX_NS;

#define NVX_FMT_DISPATCH(fmt, CALL)                                         \
    do {                                                                    \
        if ((fmt) == 0) { typedef __bf16 A_; CALL; }                        \
        else if ((fmt) == 1) { typedef _Float16 A_; CALL; }                 \
        else { typedef float A_; CALL; }                                    \
    } while (0)

extern "C" int nvx_latent_prep(const void* x, int64_t x_row_stride, int fmt, const float* w_q, const float* w_kv, float eps,
                               const int64_t* slots, void* cq, void* cache, int64_t n_slots, float* gate, int64_t n_tok, int64_t q_rank,
                               int64_t kv_rank, int64_t heads, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_latent_prep: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && q_rank > 0 && kv_rank > 0 && heads > 0 && n_slots >= 0 && q_rank + kv_rank + heads < (1 << 30) &&
                    x_row_stride >= q_rank + kv_rank + heads,
                NVX_EINVAL, "nvx_latent_prep: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && w_q && w_kv && slots && cq && cache && gate, NVX_EINVAL, "nvx_latent_prep: null pointer");
    NVX_FMT_DISPATCH(fmt, launch_prep<A_>(x, x_row_stride, w_q, w_kv, eps, slots, cq, cache, n_slots, gate, n_tok, (int)q_rank, (int)kv_rank,
                                          (int)heads, (hipStream_t)stream));
    return nvx_check_launch("nvx_latent_prep");
}

extern "C" int nvx_latent_attn(const void* q, const void* cache, int fmt, const int32_t* kv_indices, const int64_t* kv_start,
                               const int32_t* kv_len, const int32_t* qo_indptr, const int32_t* tok_seq, const float* gate, void* out,
                               int64_t heads, int64_t rank, int64_t n_tok, float scale, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_latent_attn: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && heads <= 65535 * 4 && rank > 0, NVX_EINVAL, "nvx_latent_attn: bad sizes");
    NVX_REQUIRE(rank <= 256 * LA_MAXC, NVX_EUNSUPPORTED, "nvx_latent_attn: latent size above 1024");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(q && cache && kv_indices && kv_start && kv_len && out, NVX_EINVAL, "nvx_latent_attn: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_latent_attn: tok_seq and qo_indptr go together");
    NVX_FMT_DISPATCH(fmt, launch_attn<A_>(q, cache, kv_indices, kv_start, kv_len, qo_indptr, tok_seq, gate, out, (int)heads, (int)rank, n_tok,
                                          scale, (hipStream_t)stream));
    return nvx_check_launch("nvx_latent_attn");
}
