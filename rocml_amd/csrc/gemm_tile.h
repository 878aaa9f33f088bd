// Plain tiled matrix product C[M,N] (+)= X[M,K] * W[N,K]^T for any sizes and any of the
// supported storage types, accumulating in 32-bit with fused multiply-add and no reduced-
// precision matrix instruction.  It is the whole 32-bit path's product and the fallback of
// the bfloat16 path for shapes the MFMA kernels refuse.  Tiling idea as in the reference's
// first GEMM (rocml-kernels/kernels/gemm_f16.hip:12-41), sized for a 256-thread block:
// 64x64 outputs per block, 4x4 per thread, K staged 16 at a time through LDS.
// Each output sums its K products in index order, so a row's result does not depend on
// which other rows are in the batch.
#pragma once
#include "common.h"

constexpr int GT_BM = 64, GT_BN = 64, GT_BK = 16, GT_THREADS = 256;

template <typename TX, typename TW, typename TO, bool ACCUM>
__global__ void __launch_bounds__(GT_THREADS)
gemm_tile_kernel(const TX* __restrict__ x, int ldx, const TW* __restrict__ w, int ldw,
                 TO* __restrict__ out, int ldo, int m, int n, int k) {
    __shared__ float xs[GT_BK][GT_BM + 4];
    __shared__ float ws[GT_BK][GT_BN + 4];
    int tid = threadIdx.x;
    int tx = tid % 16, ty = tid / 16;
    int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < k; k0 += GT_BK) {
        // 64 rows x 16 k = 1024 values per operand, 4 per thread; consecutive threads read
        // consecutive k of one row.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int idx = tid + i * GT_THREADS;
            int kk = idx % GT_BK, r = idx / GT_BK;
            int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
            xs[kk][r] = (gm < m && gk < k) ? Elem<TX>::load(x + (size_t)gm * ldx + gk) : 0.f;
            ws[kk][r] = (gn < n && gk < k) ? Elem<TW>::load(w + (size_t)gn * ldw + gk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int gm = m0 + ty * 4 + i;
        if (gm >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int gn = n0 + tx * 4 + j;
            if (gn >= n) continue;
            TO* p = out + (size_t)gm * ldo + gn;
            float v = acc[i][j];
            if (ACCUM) v += Elem<TO>::load(p);
            Elem<TO>::store(p, v);
        }
    }
}

template <typename TX, typename TW, typename TO>
static void launch_gemm_tile(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m,
                             int n, int k, int accumulate, hipStream_t stream) {
    dim3 grid(ceil_div(n, GT_BN), ceil_div(m, GT_BM));
    if (accumulate)
        gemm_tile_kernel<TX, TW, TO, true><<<grid, GT_THREADS, 0, stream>>>(
            (const TX*)x, ldx, (const TW*)w, ldw, (TO*)out, ldo, m, n, k);
    else
        gemm_tile_kernel<TX, TW, TO, false><<<grid, GT_THREADS, 0, stream>>>(
            (const TX*)x, ldx, (const TW*)w, ldw, (TO*)out, ldo, m, n, k);
}
