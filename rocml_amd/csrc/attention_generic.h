// Plain attention over the paged cache for any head size and either storage type: one
// 256-thread block per (query token, query head).  It serves the 32-bit path (prefill and
// decode) and every head size the fast kernels refuse.  The algebra is the reference's
// (rocml-kernels/kernels/attn_decode.hip:151-170, attn_prefill.hip:167-190): s_j = (q . k_j) *
// scale, running maximum m, l = l * e^(m - m') + sum e^(s - m'), acc likewise, out = acc / l.
// A query at position p sees keys [lo, p], lo = 0 or p - window + 1.  Keys are taken 256 at a
// time: every thread scores one key, then the threads split the head's values.
// Cache layout: keys [page, Hkv, page_size, D], values transposed in a page [page, Hkv, D, page_size].
#pragma once
#include "common.h"

constexpr int AG_BLOCK = 256;
constexpr int AG_MAX_D_PER_THREAD = 4;   // head_dim <= 1024

__device__ __forceinline__ float ag_block_max(float v, float* scratch) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < AG_BLOCK / WAVE; ++w) r = fmaxf(r, scratch[w]);
    return r;
}

__device__ __forceinline__ float ag_block_sum(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < AG_BLOCK / WAVE; ++w) r += scratch[w];
    return r;
}

template <typename T>
__global__ void __launch_bounds__(AG_BLOCK)
attn_generic_kernel(const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kcache,
                    const T* __restrict__ vcache, const int* __restrict__ block_table, int bt_width,
                    const int* __restrict__ token_seq, const int* __restrict__ token_pos, int hq,
                    int hkv, int d, int page_size, float scale, int window) {
    extern __shared__ float smem[];
    float* qs = smem;                 // [d]
    float* ps = smem + d;             // [AG_BLOCK]
    __shared__ float red[AG_BLOCK / WAVE];
    int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    int pos = token_pos[t];
    const int* pages = block_table + (size_t)token_seq[t] * bt_width;
    int kvh = h / (hq / hkv);
    int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const T* qrow = q + ((size_t)t * hq + h) * d;
    for (int e = tid; e < d; e += AG_BLOCK) qs[e] = Elem<T>::load(qrow + e);
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float acc[AG_MAX_D_PER_THREAD] = {};
    for (int c0 = lo; c0 <= pos; c0 += AG_BLOCK) {
        int j = c0 + tid;
        float s = -INFINITY;
        if (j <= pos) {
            int page = pages[j / page_size];
            const T* krow = kcache + (((size_t)page * hkv + kvh) * page_size + j % page_size) * d;
            float dot = 0.f;
            for (int e = 0; e < d; ++e) dot = fmaf(qs[e], Elem<T>::load(krow + e), dot);
            s = dot * scale;
        }
        float m_new = fmaxf(m, ag_block_max(s, red));
        float corr = expf(m - m_new);            // first chunk: exp(-inf) = 0
        float p = j <= pos ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        l = l * corr + ag_block_sum(p, red);     // barrier inside also publishes ps
        int n_keys = min(AG_BLOCK, pos - c0 + 1);
#pragma unroll
        for (int r = 0; r < AG_MAX_D_PER_THREAD; ++r) {
            int e = tid + r * AG_BLOCK;
            if (e >= d) break;
            float a = acc[r] * corr;
            for (int jj = 0; jj < n_keys; ++jj) {
                int key = c0 + jj;
                int page = pages[key / page_size];
                const T* vcol = vcache + ((size_t)page * hkv + kvh) * d * page_size + key % page_size;
                a = fmaf(ps[jj], Elem<T>::load(vcol + (size_t)e * page_size), a);
            }
            acc[r] = a;
        }
        m = m_new;
        __syncthreads();                         // ps is rewritten by the next chunk
    }
    T* orow = out + ((size_t)t * hq + h) * d;
#pragma unroll
    for (int r = 0; r < AG_MAX_D_PER_THREAD; ++r) {
        int e = tid + r * AG_BLOCK;
        if (e < d) Elem<T>::store(orow + e, acc[r] / l);
    }
}
