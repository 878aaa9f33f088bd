// Attention over the paged key/value cache for gfx950.  One entry point for any step: the
// query tokens of a step carry their sequence and position, keys and values are read from
// the cache (the step's own keys were appended before), so prefill, decode and any cut of a
// prompt run the same code.  bfloat16 with a head size that is a multiple of 32 runs on the
// matrix cores; everything else, and the whole 32-bit path, runs the plain kernel.
#include "common.h"
#include "attention_generic.h"
#include "attention_mfma.h"

ROCML_LAST_ERROR_FN(attention)

enum AttnAlgo : int { ATTN_AUTO = 0, ATTN_PLAIN = 1, ATTN_MFMA = 2 };

static const float LOG2E = 1.4426950408889634f;

template <typename K>
static int allow_lds(K kernel, int bytes) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess)
        return rocml_fail("attention: cannot reserve %d bytes of LDS: %s", bytes, hipGetErrorString(e));
    return 0;
}

struct AttnArgs {
    const bf16_t* q; bf16_t* out; const bf16_t* kcache; const bf16_t* vcache;
    const int* block_table; int bt_width; const int* token_seq; const int* token_pos;
    const int* cu_seqlens; int n_seqs; int n_tokens; int total_q_tiles; int max_len;
    int hq, hkv; float scale; int window; void* workspace; long long workspace_bytes;
    int n_splits_hint;
    const DecodeProj* proj;     // decode only: the step's q/k/v projection instead of q and an appended cache
    const PrefillProj* prefill_proj = nullptr;      // prompts: the projection instead of prepared queries
};

template <int D, bool FUSED, int AHEAD, int WAVES>
static int launch_decode_kernel(const AttnArgs& a, int n_splits, float* part_o, float* part_ml, hipStream_t stream) {
    int group = a.hq / a.hkv;
    int lds = WAVES * group * (D + 4) * (int)sizeof(float);
    static int allowed = 0;
    if (lds > allowed) {
        if (allow_lds(attn_decode_mfma_kernel<D, FUSED, AHEAD, WAVES>, lds)) return 1;
        allowed = lds;
    }
    dim3 grid(n_splits, a.hkv, a.n_tokens);
    attn_decode_mfma_kernel<D, FUSED, AHEAD, WAVES><<<grid, 64 * WAVES, lds, stream>>>(
        a.q, a.out, const_cast<bf16_t*>(a.kcache), const_cast<bf16_t*>(a.vcache), a.block_table, a.bt_width,
        a.token_seq, a.token_pos, a.hq, a.hkv, a.scale * LOG2E, a.window, n_splits, part_o, part_ml,
        FUSED ? *a.proj : DecodeProj{});
    return 0;
}

constexpr int WIDE_BLOCK_MIN_PIECES = 8;         // of a block: more than two a wave of four

template <int D, bool FUSED>
static int launch_decode(const AttnArgs& a, hipStream_t stream) {
    // Enough blocks to fill the chip, at most one split per page of the longest sequence.
    int n_splits = a.n_splits_hint;
    if (n_splits <= 0) {
        n_splits = 2 * cu_count() / (a.n_tokens * a.hkv);
        int max_pages = (a.max_len + AM_PAGE - 1) / AM_PAGE;
        if (n_splits > max_pages) n_splits = max_pages;
    }
    if (n_splits > 64) n_splits = 64;
    if (n_splits < 1) n_splits = 1;
    long long per_split = (long long)a.n_tokens * a.hq * (D + 2) * sizeof(float);
    if (n_splits > 1 && per_split * n_splits > a.workspace_bytes)
        n_splits = a.workspace ? (int)(a.workspace_bytes / per_split) : 1;
    if (n_splits < 1) n_splits = 1;
    float* part_o = (float*)a.workspace;
    float* part_ml = part_o ? part_o + (size_t)a.n_tokens * a.hq * n_splits * D : nullptr;
    // Many splits mean few pieces per block: then two of a wave's pieces travel at a time; so they
    // do when the chip holds at most one block a CU (a long loop then gains from it what a second
    // block would bring).  The choice follows the launch's shape, not the lengths, as the number of
    // splits does.
    // Eight waves a block where the chip holds at most one block a CU and a block of four waves
    // could give a wave more pieces than two trips bring (the pages the block table has room for,
    // two pieces each, over the splits and the waves: the launch's shape again, not the lengths).
    int rc;
    if constexpr (D <= 128) {
        bool one_a_cu = (long long)a.n_tokens * a.hkv * n_splits <= cu_count();
        long long pieces = 2ll * ((a.bt_width + n_splits - 1) / n_splits);
        if (one_a_cu && pieces > WIDE_BLOCK_MIN_PIECES)
            rc = launch_decode_kernel<D, FUSED, 2, 8>(a, n_splits, part_o, part_ml, stream);
        else
            rc = n_splits >= 4 || one_a_cu ? launch_decode_kernel<D, FUSED, 2, 4>(a, n_splits, part_o, part_ml, stream)
                                           : launch_decode_kernel<D, FUSED, 1, 4>(a, n_splits, part_o, part_ml, stream);
    } else {
        rc = launch_decode_kernel<D, FUSED, 1, 4>(a, n_splits, part_o, part_ml, stream);
    }
    if (rc) return rc;
    if (n_splits > 1)
        // whole waves: the kernel's reductions exchange values between all 64 lanes
        attn_decode_reduce_kernel<D><<<a.n_tokens * a.hq, (D + 63) / 64 * 64, 0, stream>>>(part_o, part_ml, a.out, n_splits);
    return 0;
}

template <int D> static int launch_decode_plain(const AttnArgs& a, hipStream_t s) { return launch_decode<D, false>(a, s); }
template <int D> static int launch_decode_fused(const AttnArgs& a, hipStream_t s) { return launch_decode<D, true>(a, s); }

template <int D>
static int launch_prefill(const AttnArgs& a, hipStream_t stream) {
    static bool ready = false;
    if (!ready) {
        if (allow_lds(attn_prefill_mfma_kernel<D, false>, PrefillLds<D>::BYTES)) return 1;
        if (allow_lds(attn_prefill_mfma_kernel<D, true>, PrefillLds<D>::BYTES)) return 1;
        ready = true;
    }
    dim3 grid(a.total_q_tiles * a.hq);
    if (a.prefill_proj)
        attn_prefill_mfma_kernel<D, true><<<grid, AM_THREADS, PrefillLds<D>::BYTES, stream>>>(
            nullptr, a.out, a.kcache, a.vcache, a.block_table, a.bt_width, a.cu_seqlens, a.n_seqs, a.token_pos,
            a.hq, a.hkv, a.scale * LOG2E, a.window, *a.prefill_proj);
    else
        attn_prefill_mfma_kernel<D, false><<<grid, AM_THREADS, PrefillLds<D>::BYTES, stream>>>(
            a.q, a.out, a.kcache, a.vcache, a.block_table, a.bt_width, a.cu_seqlens, a.n_seqs, a.token_pos,
            a.hq, a.hkv, a.scale * LOG2E, a.window, PrefillProj{});
    return 0;
}

static bool mfma_head_dim(int d) { return d == 32 || d == 64 || d == 96 || d == 128 || d == 192 || d == 256; }

#define BY_HEAD_DIM(fn, d, ...)                       \
    ((d) == 32 ? fn<32>(__VA_ARGS__)                  \
     : (d) == 64 ? fn<64>(__VA_ARGS__)                \
     : (d) == 96 ? fn<96>(__VA_ARGS__)                \
     : (d) == 128 ? fn<128>(__VA_ARGS__)              \
     : (d) == 192 ? fn<192>(__VA_ARGS__) : fn<256>(__VA_ARGS__))

// algo: 0 = choose, 1 = plain kernel, 2 = MFMA kernels (error if they cannot take the shapes).
// cu_seqlens [n_seqs + 1] gives where each sequence's query tokens start (tokens of a sequence
// are consecutive and in position order) and q_counts, an array in host memory, how many each has
// (the prefill kernel's grid is sized from it); max_new is the most query tokens of any
// sequence, max_len the longest context.
// workspace holds the partial results of split decode attention.
ROCML_EXPORT int rocml_attention(const void* q, void* out, const void* kcache, const void* vcache,
                                 int dtype, const int* block_table, int bt_width,
                                 const int* token_seq, const int* token_pos, int n_tokens, int hq,
                                 int hkv, int d, int page_size, float scale, int window, int algo,
                                 const int* cu_seqlens, int n_seqs, int max_new, const int* q_counts,
                                 int max_len, int n_splits, void* workspace, long long workspace_bytes,
                                 hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hq > 0 && hkv > 0 && d > 0 && page_size > 0 && bt_width > 0,
                  "attention: bad sizes T=%d Hq=%d Hkv=%d D=%d page=%d width=%d", n_tokens, hq, hkv,
                  d, page_size, bt_width);
    ROCML_REQUIRE(hq % hkv == 0, "attention: %d query heads are not a multiple of %d kv heads", hq, hkv);
    ROCML_REQUIRE(window >= 0, "attention: negative window %d", window);
    ROCML_REQUIRE(d <= AG_BLOCK * AG_MAX_D_PER_THREAD, "attention: head_dim %d exceeds %d", d,
                  AG_BLOCK * AG_MAX_D_PER_THREAD);
    ROCML_REQUIRE(algo >= ATTN_AUTO && algo <= ATTN_MFMA, "attention: unknown algorithm %d", algo);
    if (n_tokens == 0) return 0;
    bool decode = max_new == 1;
    long long total_q_tiles = 0, counted = 0;
    if (q_counts && n_seqs > 0)
        for (int b = 0; b < n_seqs; ++b) {
            ROCML_REQUIRE(q_counts[b] >= 0, "attention: sequence %d has %d query tokens", b, q_counts[b]);
            total_q_tiles += (q_counts[b] + AM_QTILE - 1) / AM_QTILE;
            counted += q_counts[b];
        }
    ROCML_REQUIRE(!q_counts || n_seqs <= 0 || counted == n_tokens,
                  "attention: the sequences' query counts add up to %lld, the step has %d tokens", counted, n_tokens);
    ROCML_REQUIRE(total_q_tiles * hq < (1ll << 31), "attention: too many query tiles");
    bool mfma_ok = dtype == ROCML_BF16 && page_size == AM_PAGE && mfma_head_dim(d) && max_new >= 1 &&
                   (decode ? hq / hkv <= 16 : (cu_seqlens != nullptr && n_seqs > 0 && total_q_tiles > 0));
    if (algo == ATTN_MFMA)
        ROCML_REQUIRE(mfma_ok, "attention: the MFMA kernels need bfloat16, pages of 64 positions, a head size "
                               "of 32, 64, 96, 128, 192 or 256, at most 16 query heads per kv head in decode and "
                               "the sequence offsets in prefill (D=%d page=%d group=%d)", d, page_size, hq / hkv);
    if (mfma_ok && algo != ATTN_PLAIN) {
        AttnArgs a{(const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table,
                   bt_width, token_seq, token_pos, cu_seqlens, n_seqs, n_tokens, (int)total_q_tiles, max_len, hq, hkv,
                   scale, window, workspace, workspace_bytes, n_splits, nullptr};
        int rc = decode ? BY_HEAD_DIM(launch_decode_plain, d, a, stream) : BY_HEAD_DIM(launch_prefill, d, a, stream);
        if (rc) return rc;
        ROCML_CHECK_LAUNCH("attention");
        return 0;
    }
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

// A decode step's attention straight from the q/k/v projection: per-head norm, rotation, append
// to the cache and attention in one launch (and the merge of the splits in a second), instead of
// a kernel for the first three and rocml_attention for the rest.  One token per sequence;
// bfloat16 cache with pages of 64 positions; a head size of 64, 128, 192 or 256; at most 16
// query heads per kv head.  qkv is the projection's 32-bit output [tokens, ld] with q, k and v
// side by side (k and v are not read when write_kv is 0: the cache then holds this step's row
// already), or its split-K partial sums [qkv_splits][tokens][ld], which are added in split
// order.  q_gain/k_gain null: no norm; cos/sin null: no rotation, else [tokens, D/2].
// token_seq null: token t is the one token of the step's sequence t (row t of the block table).
// row_ssq (may be null): the projection's operand lacked its norm's scale (see DecodeProj).
ROCML_EXPORT int rocml_attention_decode_fused(const float* qkv, int ld, int qkv_splits, long long qkv_split_stride,
                                              const float* q_gain, const float* k_gain, float eps,
                                              const float* cos_t, const float* sin_t, int write_kv, void* out,
                                              void* kcache, void* vcache, const int* block_table, int bt_width,
                                              const int* token_seq, const int* token_pos, int n_tokens, int hq,
                                              int hkv, int d, int page_size, float scale, int window,
                                              int max_len, int n_splits, void* workspace,
                                              long long workspace_bytes, const float* row_ssq, int row_parts,
                                              float row_eps, int row_width, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hq > 0 && hkv > 0 && bt_width > 0 && qkv_splits >= 1,
                  "fused decode attention: bad sizes T=%d Hq=%d Hkv=%d width=%d splits=%d", n_tokens, hq, hkv,
                  bt_width, qkv_splits);
    ROCML_REQUIRE(hq % hkv == 0 && hq / hkv <= 16,
                  "fused decode attention: %d query heads over %d kv heads (at most 16 per kv head)", hq, hkv);
    ROCML_REQUIRE(page_size == AM_PAGE && (d == 64 || d == 128 || d == 192 || d == 256),
                  "fused decode attention: needs pages of 64 positions and a head size of 64, 128, 192 or 256 "
                  "(page=%d D=%d)", page_size, d);
    ROCML_REQUIRE(window >= 0, "fused decode attention: negative window %d", window);
    int rows = write_kv ? hq + 2 * hkv : hq;
    ROCML_REQUIRE(ld >= rows * d && ld % 4 == 0 && ((uintptr_t)qkv & 15) == 0 &&
                      (qkv_splits == 1 || (qkv_split_stride >= (long long)n_tokens * ld && qkv_split_stride % 4 == 0)),
                  "fused decode attention: projection rows of %d values (need %d, a multiple of 4, 16-byte aligned), "
                  "split stride %lld", ld, rows * d, qkv_split_stride);
    ROCML_REQUIRE((q_gain == nullptr) == (k_gain == nullptr) && (cos_t == nullptr) == (sin_t == nullptr),
                  "fused decode attention: gains and rotation tables come in pairs");
    if (n_tokens == 0) return 0;
    ROCML_REQUIRE(!row_ssq || (row_parts > 0 && row_eps > 0.f && row_width > 0),
                  "fused decode attention: a row scale needs parts, eps and the norm's width");
    DecodeProj pj{qkv, ld, qkv_splits, qkv_split_stride, q_gain, k_gain, eps, cos_t, sin_t, write_kv,
                  row_ssq, row_parts, row_eps, row_ssq ? 1.0f / (float)row_width : 0.f};
    AttnArgs a{nullptr, (bf16_t*)out, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table, bt_width,
               token_seq, token_pos, nullptr, 0, n_tokens, 0, max_len, hq, hkv, scale, window, workspace,
               workspace_bytes, n_splits, &pj};
    int rc = d == 64 ? launch_decode_fused<64>(a, stream)
             : d == 128 ? launch_decode_fused<128>(a, stream)
             : d == 192 ? launch_decode_fused<192>(a, stream) : launch_decode_fused<256>(a, stream);
    if (rc) return rc;
    ROCML_CHECK_LAUNCH("fused decode attention");
    return 0;
}

// Prompts: attention of a step's new tokens over the cache, with the queries taken from the step's
// q/k/v projection (32-bit, complete sums: a token's q heads first) and prepared by the kernel
// itself: per-head norm (q_gain null: none), rotation of the whole head with pairs (e, e + D/2)
// (cos/sin null: none, else [tokens, D/2]), rounding to bfloat16.  The keys and values of the new
// tokens are in the cache already.  bfloat16 caches with pages of 64 positions and the MFMA
// kernels' head sizes; cu_seqlens, q_counts as in rocml_attention.
ROCML_EXPORT int rocml_attention_prefill_fused(const float* qkv, int ld, const float* q_gain, float eps,
                                               const float* cos_t, const float* sin_t, void* out,
                                               const void* kcache, const void* vcache, const int* block_table,
                                               int bt_width, const int* token_pos, int n_tokens, int hq, int hkv,
                                               int d, int page_size, float scale, int window,
                                               const int* cu_seqlens, int n_seqs, const int* q_counts,
                                               hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hq > 0 && hkv > 0 && bt_width > 0 && n_seqs > 0 && cu_seqlens && q_counts,
                  "fused prefill attention: bad sizes T=%d Hq=%d Hkv=%d width=%d sequences=%d", n_tokens, hq, hkv,
                  bt_width, n_seqs);
    ROCML_REQUIRE(hq % hkv == 0, "fused prefill attention: %d query heads are not a multiple of %d kv heads", hq, hkv);
    ROCML_REQUIRE(page_size == AM_PAGE && mfma_head_dim(d),
                  "fused prefill attention: needs pages of 64 positions and a head size of 32, 64, 96, 128, 192 or 256 "
                  "(page=%d D=%d)", page_size, d);
    ROCML_REQUIRE(window >= 0, "fused prefill attention: negative window %d", window);
    ROCML_REQUIRE(ld >= hq * d && ld % 4 == 0 && ((uintptr_t)qkv & 15) == 0,
                  "fused prefill attention: projection rows of %d values (need %d, a multiple of 4, 16-byte aligned)",
                  ld, hq * d);
    ROCML_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "fused prefill attention: rotation tables come in pairs");
    ROCML_REQUIRE(!q_gain || ((uintptr_t)q_gain & 15) == 0, "fused prefill attention: the gain must be 16-byte aligned");
    ROCML_REQUIRE(!cos_t || ((((uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0),
                  "fused prefill attention: the rotation tables must be 16-byte aligned");
    if (n_tokens == 0) return 0;
    long long total_q_tiles = 0, counted = 0;
    for (int b = 0; b < n_seqs; ++b) {
        ROCML_REQUIRE(q_counts[b] >= 0, "fused prefill attention: sequence %d has %d query tokens", b, q_counts[b]);
        total_q_tiles += (q_counts[b] + AM_QTILE - 1) / AM_QTILE;
        counted += q_counts[b];
    }
    ROCML_REQUIRE(counted == n_tokens, "fused prefill attention: the sequences' query counts add up to %lld, the step has %d tokens",
                  counted, n_tokens);
    ROCML_REQUIRE(total_q_tiles > 0 && total_q_tiles * hq < (1ll << 31), "fused prefill attention: %lld query tiles", total_q_tiles);
    PrefillProj pj{qkv, ld, q_gain, eps, cos_t, sin_t};
    AttnArgs a{nullptr, (bf16_t*)out, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table, bt_width,
               nullptr, token_pos, cu_seqlens, n_seqs, n_tokens, (int)total_q_tiles, 0, hq, hkv, scale, window, nullptr,
               0, 0, nullptr};
    a.prefill_proj = &pj;
    int rc = BY_HEAD_DIM(launch_prefill, d, a, stream);
    if (rc) return rc;
    ROCML_CHECK_LAUNCH("fused prefill attention");
    return 0;
}
