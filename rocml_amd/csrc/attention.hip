// Attention over the paged key/value cache for gfx950.  One entry point for any step: the
// query tokens of a step carry their sequence and position, keys and values are read from
// the cache (the step's own keys were appended before), so prefill, decode and any cut of a
// prompt run the same code.
#include "common.h"
#include "attention_generic.h"

ROCML_LAST_ERROR_FN(attention)

// algo: 0 = choose, 1 = plain kernel.
ROCML_EXPORT int rocml_attention(const void* q, void* out, const void* kcache, const void* vcache,
                                 int dtype, const int* block_table, int bt_width,
                                 const int* token_seq, const int* token_pos, int n_tokens, int hq,
                                 int hkv, int d, int page_size, float scale, int window, int algo,
                                 void* workspace, long long workspace_bytes, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hq > 0 && hkv > 0 && d > 0 && page_size > 0 && bt_width > 0,
                  "attention: bad sizes T=%d Hq=%d Hkv=%d D=%d page=%d width=%d", n_tokens, hq, hkv,
                  d, page_size, bt_width);
    ROCML_REQUIRE(hq % hkv == 0, "attention: %d query heads are not a multiple of %d kv heads", hq, hkv);
    ROCML_REQUIRE(window >= 0, "attention: negative window %d", window);
    ROCML_REQUIRE(d <= AG_BLOCK * AG_MAX_D_PER_THREAD, "attention: head_dim %d exceeds %d", d,
                  AG_BLOCK * AG_MAX_D_PER_THREAD);
    (void)algo; (void)workspace; (void)workspace_bytes;
    if (n_tokens == 0) return 0;
    dim3 grid(n_tokens, hq);
    size_t lds = (size_t)(d + AG_BLOCK) * sizeof(float);
    if (dtype == ROCML_F32)
        attn_generic_kernel<float><<<grid, AG_BLOCK, lds, stream>>>(
            (const float*)q, (float*)out, (const float*)kcache, (const float*)vcache, block_table,
            bt_width, token_seq, token_pos, hq, hkv, d, page_size, scale, window);
    else if (dtype == ROCML_BF16)
        attn_generic_kernel<bf16_t><<<grid, AG_BLOCK, lds, stream>>>(
            (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table,
            bt_width, token_seq, token_pos, hq, hkv, d, page_size, scale, window);
    else
        return rocml_fail("attention: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("attention");
    return 0;
}
