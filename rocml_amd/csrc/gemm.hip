// Matrix products of the decoder: out[M,N] (+)= X[M,K] * W[N,K]^T, weights row-major
// [out, in] as the reference keeps them (rocml/src/weights/mod.rs:78-98).
#include "common.h"
#include "gemm_tile.h"

ROCML_LAST_ERROR_FN(gemm)

// algo: 0 = choose, 1 = plain tiled kernel.
// accumulate: out += product (out must be 32-bit); this is the residual sum's epilogue.
ROCML_EXPORT int rocml_gemm(const void* x, int x_dtype, int ldx, const void* w, int w_dtype, int ldw,
                            void* out, int out_dtype, int ldo, int m, int n, int k, int accumulate,
                            int algo, void* workspace, long long workspace_bytes,
                            hipStream_t stream) {
    ROCML_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm: bad sizes M=%d N=%d K=%d", m, n, k);
    ROCML_REQUIRE(ldx >= k && ldw >= k && ldo >= n, "gemm: row strides (%d, %d, %d) below (K, K, N)",
                  ldx, ldw, ldo);
    ROCML_REQUIRE(!accumulate || out_dtype == ROCML_F32, "gemm: accumulation needs a 32-bit output");
    (void)algo; (void)workspace; (void)workspace_bytes;
    if (m == 0) return 0;
    if (x_dtype == ROCML_F32 && w_dtype == ROCML_F32 && out_dtype == ROCML_F32)
        launch_gemm_tile<float, float, float>(x, ldx, w, ldw, out, ldo, m, n, k, accumulate, stream);
    else if (x_dtype == ROCML_BF16 && w_dtype == ROCML_BF16 && out_dtype == ROCML_F32)
        launch_gemm_tile<bf16_t, bf16_t, float>(x, ldx, w, ldw, out, ldo, m, n, k, accumulate, stream);
    else if (x_dtype == ROCML_BF16 && w_dtype == ROCML_BF16 && out_dtype == ROCML_BF16)
        launch_gemm_tile<bf16_t, bf16_t, bf16_t>(x, ldx, w, ldw, out, ldo, m, n, k, 0, stream);
    else
        return rocml_fail("gemm: unsupported dtype triple x=%d w=%d out=%d", x_dtype, w_dtype, out_dtype);
    ROCML_CHECK_LAUNCH("gemm");
    return 0;
}
