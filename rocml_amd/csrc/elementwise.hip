// Memory-bound kernels of the decoder for gfx950 (wave64): embedding gather, RMSNorm,
// SwiGLU, rotation tables, and the fused per-head norm + rotation + cache append.
// Norm statistics, angles and the SiLU are computed in 32-bit (angles in 64-bit) whatever
// the storage type is.
#include "common.h"

ROCML_LAST_ERROR_FN(elementwise)

constexpr int EW_BLOCK = 256;

// ---- embedding -------------------------------------------------------------------
// out[t, :] = float(table[ids[t], :]) * scale  (rocml-kernels/kernels/embedding.hip:6-18;
// the reference has no scale, callers pass 1).
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, int vocab, float scale) {
    int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + (size_t)id * hidden;
    float* o = out + (size_t)t * hidden;
    for (int i = threadIdx.x; i < hidden; i += EW_BLOCK) o[i] = Elem<T>::load(row + i) * scale;
}

ROCML_EXPORT int rocml_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                                    int n_tokens, int hidden, int vocab, float scale,
                                    hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes T=%d H=%d V=%d",
                  n_tokens, hidden, vocab);
    if (n_tokens == 0) return 0;
    if (table_dtype == ROCML_F32)
        embed_gather_kernel<float><<<n_tokens, EW_BLOCK, 0, stream>>>((const float*)table, ids, out,
                                                                      hidden, vocab, scale);
    else if (table_dtype == ROCML_BF16)
        embed_gather_kernel<bf16_t><<<n_tokens, EW_BLOCK, 0, stream>>>((const bf16_t*)table, ids, out,
                                                                       hidden, vocab, scale);
    else
        return rocml_fail("embed_gather: unknown dtype code %d", table_dtype);
    ROCML_CHECK_LAUNCH("embed_gather");
    return 0;
}

// ---- block reduction -------------------------------------------------------------
// Sum over a block of EW_BLOCK threads in a fixed order: lanes by butterfly, waves in order.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    int wave = threadIdx.x / WAVE;
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < EW_BLOCK / WAVE; ++w) total += scratch[w];
    return total;
}

// ---- RMSNorm ---------------------------------------------------------------------
// out[r, i] = x[src(r), i] * (1/sqrt(sum(x^2)/n + eps)) * gain[i]
// (rocml-kernels/kernels/rmsnorm.hip:18-42).  `rows` optionally gathers source rows.
// With `partials` ([n_splits][rows of x][n], the split-K partial sums of the product whose
// result belongs to x) the kernel first forms x + sum of the partials in split order, which is
// the residual sum the reference does in a kernel of its own
// (rocml-kernels/kernels/elementwise.hip:7-12), writes it back to x unless rows are gathered,
// and normalises that.
template <typename TO>
__global__ void rmsnorm_kernel(float* x, const float* __restrict__ gain, TO* __restrict__ out,
                               const int* __restrict__ rows, int n, float eps,
                               const float* __restrict__ partials, int n_splits, long long split_stride) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    int r = blockIdx.x;
    int src = rows ? rows[r] : r;
    float* xin = x + (size_t)src * n;
    TO* o = out + (size_t)r * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float v = xin[i];
        for (int sp = 0; sp < n_splits; ++sp) v += partials[sp * split_stride + (size_t)src * n + i];
        if (n_splits > 0 && !rows) xin[i] = v;
        ss = fmaf(v, v, ss);
    }
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float v = xin[i];
        if (rows) for (int sp = 0; sp < n_splits; ++sp) v += partials[sp * split_stride + (size_t)src * n + i];
        Elem<TO>::store(o + i, v * inv * gain[i]);
    }
}

// Same result for rows of up to 8192 values that are a multiple of 4: the row stays in
// registers between the two passes and all loads are issued at once (a loop of single loads
// waits for each one in turn, which is what a one-row decode step would spend its time on).
constexpr int RN_MAX_VEC = 8;

__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    *(float4*)p = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
    uint2 v;
    v.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    v.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *(uint2*)p = v;
}

template <typename TO, int RN_VEC>
__global__ void __launch_bounds__(EW_BLOCK)
rmsnorm_vec_kernel(float* x, const float* __restrict__ gain, TO* __restrict__ out,
                   const int* __restrict__ rows, int n, float eps, const float* __restrict__ partials,
                   int n_splits, long long split_stride) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    int r = blockIdx.x;
    int src = rows ? rows[r] : r;
    float4* xin = (float4*)(x + (size_t)src * n);
    const float4* g4 = (const float4*)gain;
    TO* o = out + (size_t)r * n;
    int nv = n / 4;
    float4 v[RN_VEC], g[RN_VEC];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j) {
        int idx = threadIdx.x + j * EW_BLOCK;
        bool ok = idx < nv;
        v[j] = xin[ok ? idx : 0];
        g[j] = g4[ok ? idx : 0];
        if (!ok) v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (n_splits > 0) {
        const float4* p4 = (const float4*)(partials + (size_t)src * n);
        long long stride4 = split_stride / 4;
        constexpr int GROUP = 32 / RN_VEC;              // splits whose loads are in flight together
        for (int sp = 0; sp < n_splits; sp += GROUP) {  // loads of a group all issued, added in split order
            float4 a[GROUP][RN_VEC];
#pragma unroll
            for (int q = 0; q < GROUP; ++q)
#pragma unroll
                for (int j = 0; j < RN_VEC; ++j) {
                    int idx = threadIdx.x + j * EW_BLOCK;
                    int safe = idx < nv ? idx : 0;
                    a[q][j] = p4[(sp + q < n_splits ? sp + q : sp) * stride4 + safe];
                }
#pragma unroll
            for (int q = 0; q < GROUP; ++q)
#pragma unroll
                for (int j = 0; j < RN_VEC; ++j) {
                    if ((int)threadIdx.x + j * EW_BLOCK >= nv || sp + q >= n_splits) continue;
                    v[j].x += a[q][j].x; v[j].y += a[q][j].y; v[j].z += a[q][j].z; v[j].w += a[q][j].w;
                }
        }
        if (!rows) {
#pragma unroll
            for (int j = 0; j < RN_VEC; ++j) {
                int idx = threadIdx.x + j * EW_BLOCK;
                if (idx < nv) xin[idx] = v[j];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j)
        ss = fmaf(v[j].x, v[j].x, fmaf(v[j].y, v[j].y, fmaf(v[j].z, v[j].z, fmaf(v[j].w, v[j].w, ss))));
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / (float)n + eps);
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j) {
        int idx = threadIdx.x + j * EW_BLOCK;
        if (idx < nv)
            store4(o + 4 * idx, v[j].x * inv * g[j].x, v[j].y * inv * g[j].y, v[j].z * inv * g[j].z,
                   v[j].w * inv * g[j].w);
    }
}

ROCML_EXPORT int rocml_rmsnorm(float* x, const float* gain, void* out, int out_dtype, const int* rows,
                               int n_rows, int n, float eps, const float* partials, int n_splits,
                               long long split_stride, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0, "rmsnorm: bad sizes rows=%d n=%d", n_rows, n);
    ROCML_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive, got %g", (double)eps);
    ROCML_REQUIRE(n_splits >= 0 && (n_splits == 0 || (partials && split_stride > 0)),
                  "rmsnorm: partial sums need a pointer and a stride");
    if (n_rows == 0) return 0;
    bool vec = n % 4 == 0 && n <= 4 * RN_MAX_VEC * EW_BLOCK && (uintptr_t)x % 16 == 0 &&
               (uintptr_t)gain % 16 == 0 && (uintptr_t)out % 16 == 0 &&
               (n_splits == 0 || ((uintptr_t)partials % 16 == 0 && split_stride % 4 == 0));
#define RN_ARGS rows, n, eps, partials, n_splits, split_stride
    bool small = n <= 4 * 4 * EW_BLOCK;      // rows of up to 4096 values: 4 vectors per thread
    if (vec && out_dtype == ROCML_F32 && small)
        rmsnorm_vec_kernel<float, 4><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_F32)
        rmsnorm_vec_kernel<float, 8><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_BF16 && small)
        rmsnorm_vec_kernel<bf16_t, 4><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_BF16)
        rmsnorm_vec_kernel<bf16_t, 8><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else if (out_dtype == ROCML_F32)
        rmsnorm_kernel<float><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (out_dtype == ROCML_BF16)
        rmsnorm_kernel<bf16_t><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else
        return rocml_fail("rmsnorm: unknown dtype code %d", out_dtype);
#undef RN_ARGS
    ROCML_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// ---- gated activation ------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i],  silu(g) = g / (1 + exp(-g))
// (rocml-kernels/kernels/silu_mul.hip:12-20).  Gate and up halves lie side by side in a row.
// With `interleaved` a row holds (gate_0, up_0, gate_1, up_1, ...), the order the fused product
// epilogue wants its weight rows in.
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter,
                              long long total, int interleaved) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / inter;
    int i = (int)(idx - t * inter);
    const TI* row = gu + (size_t)t * 2 * inter;
    float g = Elem<TI>::load(row + (interleaved ? 2 * i : i));
    float u = Elem<TI>::load(row + (interleaved ? 2 * i + 1 : inter + i));
    Elem<TO>::store(out + idx, g / (1.0f + expf(-g)) * u);
}

ROCML_EXPORT int rocml_swiglu(const void* gu, int in_dtype, void* out, int out_dtype, int n_tokens,
                              int inter, int interleaved, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", n_tokens, inter);
    long long total = (long long)n_tokens * inter;
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (in_dtype == ROCML_F32 && out_dtype == ROCML_F32)
        swiglu_kernel<float, float><<<grid, EW_BLOCK, 0, stream>>>((const float*)gu, (float*)out, inter, total, interleaved);
    else if (in_dtype == ROCML_F32 && out_dtype == ROCML_BF16)
        swiglu_kernel<float, bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const float*)gu, (bf16_t*)out, inter, total, interleaved);
    else if (in_dtype == ROCML_BF16 && out_dtype == ROCML_BF16)
        swiglu_kernel<bf16_t, bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter, total, interleaved);
    else
        return rocml_fail("swiglu: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
    ROCML_CHECK_LAUNCH("swiglu");
    return 0;
}

// ---- rotation tables -------------------------------------------------------------
// cos/sin of pos * inv_freq[i] for every token of a step, angle formed in 64-bit so that the
// 32-bit table is exact to rounding (the reference forms the angle in 32-bit,
// rocml-kernels/kernels/rope.hip:23-27).  inv_freq[i] = theta^(-2i/rot_dim) comes from the host.
__global__ void rope_table_kernel(const int* __restrict__ pos, const double* __restrict__ inv_freq,
                                  float* __restrict__ cos_t, float* __restrict__ sin_t, int half,
                                  long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / half;
    int i = (int)(idx - t * half);
    double a = (double)pos[t] * inv_freq[i];
    cos_t[idx] = (float)cos(a);
    sin_t[idx] = (float)sin(a);
}

ROCML_EXPORT int rocml_rope_table(const int* pos, const double* inv_freq, float* cos_t, float* sin_t,
                                  int n_tokens, int half, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && half > 0, "rope_table: bad sizes T=%d half=%d", n_tokens, half);
    long long total = (long long)n_tokens * half;
    if (total == 0) return 0;
    rope_table_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(pos, inv_freq, cos_t, sin_t,
                                                                           half, total);
    ROCML_CHECK_LAUNCH("rope_table");
    return 0;
}

// ---- per-head norm + rotation + cache append -------------------------------------
// One wave per (token, head row) of the packed projection output [T, (Hq + 2 Hkv) * D]:
// q and k rows are normalised over D with one gain vector each
// (rocml/src/forward/attention.rs:105-123), rotated with NEOX pairing (i, i + rot/2)
// (rocml-kernels/kernels/rope.hip:18-33); with n_splits > 1 the input is the projection's split-K
// partial sums [n_splits][T, ld], summed here in split order; q goes to q_out, k and v go straight into the
// paged cache at the token's position (rocml-kernels/kernels/chunk_reshape.hip:37-74 is the
// reference's separate scatter).  Cache layout: keys [page, Hkv, page_size, D], values
// transposed inside a page [page, Hkv, D, page_size] (what the MFMA attention kernels read).
constexpr int QK_MAX_PER_LANE = 8;   // D <= 512
constexpr int QK_WAVES = EW_BLOCK / WAVE;

// LOCAL_PAIR: the whole head is rotated and a lane holds at least two values, so both values of a
// pair (e, e + d/2) are in the same lane and no exchange through LDS is needed.
template <typename TI, typename TO, int QK_PER_LANE, bool LOCAL_PAIR>
__global__ void qk_norm_rope_append_kernel(
    const TI* __restrict__ qkv, int ld, int n_tokens, int hq, int hkv, int d,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
    TO* __restrict__ q_out, TO* __restrict__ kcache, TO* __restrict__ vcache,
    const int* __restrict__ block_table, int bt_width, const int* __restrict__ token_seq,
    const int* __restrict__ token_pos, int page_size, int write_kv, int n_splits, long long split_stride,
    int rows_per_token, int pairing, int first_row) {
    extern __shared__ float stage[];   // [QK_WAVES][d]
    int wave = threadIdx.x / WAVE;
    int lane = threadIdx.x & (WAVE - 1);
    long long row = (long long)blockIdx.x * QK_WAVES + wave;
    bool active = row < (long long)n_tokens * rows_per_token;
    int t = active ? (int)(row / rows_per_token) : 0;
    int r = first_row + (active ? (int)(row - (long long)t * rows_per_token) : 0);     // first_row = hq: no q rows
    int kind = r < hq ? 0 : (r < hq + hkv ? 1 : 2);   // q, k, v
    if (!write_kv && kind != 0) active = false;
    const TI* src = qkv + (size_t)t * ld + (size_t)r * d;
    float v[QK_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QK_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        bool ok = active && e < d;
        float val = Elem<TI>::load(ok ? src + e : qkv);
        // split-K partial sums of the projection, added in split order
        // (four loads in flight at a time)
        for (int sp = 1; sp < n_splits; sp += 4) {
            const TI* p = ok ? src + e : qkv;
            float a0 = Elem<TI>::load(ok ? p + sp * split_stride : qkv);
            float a1 = Elem<TI>::load(ok && sp + 1 < n_splits ? p + (sp + 1) * split_stride : qkv);
            float a2 = Elem<TI>::load(ok && sp + 2 < n_splits ? p + (sp + 2) * split_stride : qkv);
            float a3 = Elem<TI>::load(ok && sp + 3 < n_splits ? p + (sp + 3) * split_stride : qkv);
            val += a0;
            if (sp + 1 < n_splits) val += a1;
            if (sp + 2 < n_splits) val += a2;
            if (sp + 3 < n_splits) val += a3;
        }
        v[j] = ok ? val : 0.f;
        ss = fmaf(v[j], v[j], ss);
    }
    const float* gain = kind == 0 ? q_gain : (kind == 1 ? k_gain : nullptr);
    if (gain) {
        float inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) {
            int e = lane + j * WAVE;
            if (e < d) v[j] = v[j] * inv * gain[e];
        }
    }
    bool rotate = cos_t != nullptr && kind != 2;
    if (LOCAL_PAIR) {
        if (rotate) {
            constexpr int HJ = QK_PER_LANE / 2 > 0 ? QK_PER_LANE / 2 : 1;
            const float* c = cos_t + (size_t)t * (d / 2);
            const float* s = sin_t + (size_t)t * (d / 2);
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                int e = lane + j * WAVE;                     // pair (e, e + d/2) = values j and j + HJ
                float cs = c[e], sn = s[e], lo = v[j], hi = v[j + HJ];
                v[j] = lo * cs - hi * sn;
                v[j + HJ] = lo * sn + hi * cs;
            }
        }
    } else {
        float* mine = stage + (size_t)wave * d;
        if (rotate) {
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < d) mine[e] = v[j];
            }
        }
        __syncthreads();
        if (rotate) {
            int half = rot / 2;
            const float* c = cos_t + (size_t)t * half;
            const float* s = sin_t + (size_t)t * half;
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < rot) {
                    if (pairing == 1) {
                        // neighbours (2i, 2i + 1) are a pair, angle i
                        float cs = c[e >> 1], sn = s[e >> 1], other = mine[e ^ 1];
                        v[j] = (e & 1) ? other * sn + v[j] * cs : v[j] * cs - other * sn;
                    } else if (e < half) {
                        v[j] = v[j] * c[e] - mine[e + half] * s[e];
                    } else {
                        v[j] = mine[e - half] * s[e - half] + v[j] * c[e - half];
                    }
                }
            }
        }
    }
    if (!active) return;
    TO* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)t * hq + r) * d;
    } else {
        int head = kind == 1 ? r - hq : r - hq - hkv;
        int pos = token_pos[t];
        int page = block_table[(size_t)token_seq[t] * bt_width + pos / page_size];
        if (page < 0) return;
        if (kind == 2) {
            // values are stored transposed inside a page: [page, Hkv, D, page_size]
            TO* vdst = vcache + ((size_t)page * hkv + head) * d * page_size + pos % page_size;
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < d) Elem<TO>::store(vdst + (size_t)e * page_size, v[j]);
            }
            return;
        }
        dst = kcache + (((size_t)page * hkv + head) * page_size + pos % page_size) * d;
    }
#pragma unroll
    for (int j = 0; j < QK_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        if (e < d) Elem<TO>::store(dst + e, v[j]);
    }
}

// Prompts: q and k rows of many tokens.  A wave takes ROWS rows and issues the loads of all of
// them before it works on the first (one row per wave leaves too few bytes in flight and too
// many tiny blocks to dispatch).  Only the case LOCAL_PAIR describes: whole head rotated, both
// values of a pair in one lane, complete projections (no partial sums).
template <typename TI, typename TO, int QK_PER_LANE, int ROWS>
__global__ void __launch_bounds__(EW_BLOCK)
qk_norm_rope_rows_kernel(
    const TI* __restrict__ qkv, int ld, int n_tokens, int hq, int hkv, int d,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    TO* __restrict__ q_out, TO* __restrict__ kcache, const int* __restrict__ block_table, int bt_width,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos, int page_size, int rows_per_token,
    int first_row) {
    constexpr int HJ = QK_PER_LANE / 2;
    int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
    long long total = (long long)n_tokens * rows_per_token;
    long long row0 = ((long long)blockIdx.x * QK_WAVES + wave) * ROWS;
    float v[ROWS][QK_PER_LANE], cs[ROWS][HJ], sn[ROWS][HJ];
    int tok[ROWS], rr[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        long long row = min(row0 + i, total - 1);            // rows past the end repeat the last one, not stored
        tok[i] = (int)(row / rows_per_token);
        rr[i] = first_row + (int)(row - (long long)tok[i] * rows_per_token);
        const TI* src = qkv + (size_t)tok[i] * ld + (size_t)rr[i] * d;
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] = Elem<TI>::load(src + lane + j * WAVE);
        if (cos_t) {
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                cs[i][j] = cos_t[(size_t)tok[i] * (d / 2) + lane + j * WAVE];
                sn[i][j] = sin_t[(size_t)tok[i] * (d / 2) + lane + j * WAVE];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        bool is_q = rr[i] < hq;
        const float* gain = is_q ? q_gain : k_gain;
        if (gain) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) ss = fmaf(v[i][j], v[i][j], ss);
            float inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] = v[i][j] * inv * gain[lane + j * WAVE];
        }
        if (cos_t) {
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                float lo = v[i][j], hi = v[i][j + HJ];
                v[i][j] = lo * cs[i][j] - hi * sn[i][j];
                v[i][j + HJ] = lo * sn[i][j] + hi * cs[i][j];
            }
        }
        if (row0 + i >= total) continue;
        TO* dst;
        if (is_q) {
            dst = q_out + ((size_t)tok[i] * hq + rr[i]) * d;
        } else {
            int pos = token_pos[tok[i]];
            int page = block_table[(size_t)token_seq[tok[i]] * bt_width + pos / page_size];
            if (page < 0) continue;
            dst = kcache + (((size_t)page * hkv + (rr[i] - hq)) * page_size + pos % page_size) * d;
        }
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) Elem<TO>::store(dst + lane + j * WAVE, v[i][j]);
    }
}

// Values of many tokens at once (prompts): a block takes 64 consecutive tokens of the packed
// batch, one key/value head and 32 of its values, stages them in LDS and writes them transposed.
// In the transposed page a token is one 2- or 4-byte column; written token by token every store
// would touch a cache line of its own, written this way the 64 lanes of a wave store 64
// neighbouring positions of one row (they are neighbours wherever the tokens are consecutive
// positions of one sequence inside one page, which is the rule in a prompt).
constexpr int VT_TOKENS = 64, VT_VALUES = 32;

template <typename TI, typename TO>
__global__ void __launch_bounds__(EW_BLOCK)
v_append_tile_kernel(const TI* __restrict__ qkv, int ld, int n_tokens, int v_col0, int hkv, int d,
                     TO* __restrict__ vcache, const int* __restrict__ block_table, int bt_width,
                     const int* __restrict__ token_seq, const int* __restrict__ token_pos, int page_size) {
    __shared__ float vt_stage[VT_TOKENS][VT_VALUES + 1];
    int t0 = blockIdx.x * VT_TOKENS, head = blockIdx.y, e0 = blockIdx.z * VT_VALUES;
    int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    // thread -> (token tid/32 + 8*i, value tid%32): 128 contiguous bytes per token row
    float tmp[VT_TOKENS * VT_VALUES / EW_BLOCK];
#pragma unroll
    for (int i = 0; i < VT_TOKENS * VT_VALUES / EW_BLOCK; ++i) {
        int j = min(t0 + (tid >> 5) + (EW_BLOCK / VT_VALUES) * i, n_tokens - 1), e = min(e0 + (tid & 31), d - 1);
        tmp[i] = Elem<TI>::load(qkv + (size_t)j * ld + v_col0 + (size_t)head * d + e);
    }
#pragma unroll
    for (int i = 0; i < VT_TOKENS * VT_VALUES / EW_BLOCK; ++i) vt_stage[(tid >> 5) + (EW_BLOCK / VT_VALUES) * i][tid & 31] = tmp[i];
    __syncthreads();
    int t = t0 + lane;
    if (t >= n_tokens) return;
    int pos = token_pos[t];
    int page = block_table[(size_t)token_seq[t] * bt_width + pos / page_size];
    if (page < 0) return;
    TO* dst = vcache + ((size_t)page * hkv + head) * d * page_size + pos % page_size;
#pragma unroll
    for (int i = 0; i < VT_VALUES / (EW_BLOCK / WAVE); ++i) {
        int el = wave + (EW_BLOCK / WAVE) * i;
        if (e0 + el < d) Elem<TO>::store(dst + (size_t)(e0 + el) * page_size, vt_stage[lane][el]);
    }
}

ROCML_EXPORT int rocml_qk_norm_rope_append(
    const void* qkv, int in_dtype, int ld, int n_tokens, int hq, int hkv, int d, const float* q_gain,
    const float* k_gain, float eps, const float* cos_t, const float* sin_t, int rot, int pairing, void* q_out,
    void* kcache, void* vcache, int out_dtype, const int* block_table, int bt_width,
    const int* token_seq, const int* token_pos, int page_size, int write_kv, int n_splits,
    long long split_stride, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hq > 0 && hkv > 0 && d > 0, "qk_norm_rope_append: bad sizes");
    ROCML_REQUIRE(n_splits >= 1 && (n_splits == 1 || (split_stride > 0 && in_dtype == ROCML_F32)),
                  "qk_norm_rope_append: partial sums must be 32-bit with a positive stride");
    ROCML_REQUIRE(d <= QK_MAX_PER_LANE * WAVE, "qk_norm_rope_append: head_dim %d exceeds %d", d,
                  QK_MAX_PER_LANE * WAVE);
    ROCML_REQUIRE(ld >= (hq + 2 * hkv) * d || (!write_kv && ld >= hq * d),
                  "qk_norm_rope_append: row stride %d too small", ld);
    ROCML_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "qk_norm_rope_append: rot_dim %d must be even and <= %d", rot, d);
    ROCML_REQUIRE(pairing == 0 || pairing == 1, "qk_norm_rope_append: pairing %d (0: halves, 1: neighbours)", pairing);
    ROCML_REQUIRE(!write_kv || (page_size > 0 && bt_width > 0 && block_table && kcache && vcache),
                  "qk_norm_rope_append: cache arguments missing");
    ROCML_REQUIRE(q_out || write_kv, "qk_norm_rope_append: nothing to write");
    if (n_tokens == 0) return 0;
    // prompts: the values go through the transposing tile kernel, the row kernel does q and k
    bool v_tiled = write_kv && n_splits == 1 && n_tokens >= VT_TOKENS;
    // (without q_out the q rows are left to the caller: the prefill attention that reads the
    // projection prepares its queries itself)
    int first_row = q_out ? 0 : hq;
    int rows_per_token = hq - first_row + (write_kv ? (v_tiled ? hkv : 2 * hkv) : 0);
    long long rows = (long long)n_tokens * rows_per_token;
    int per_lane = d <= 64 ? 1 : d <= 128 ? 2 : d <= 256 ? 4 : 8;     // head values per lane
    // both values of a rotation pair in one lane: whole head rotated, d = per_lane * 64
    // (and the pairs are (e, e + d/2): neighbours as pairs go through LDS)
    bool local_pair = per_lane >= 2 && (rot == 0 || (rot == d && pairing == 0)) && d == per_lane * WAVE;
    // many rows, none of them values: several rows per wave
    bool many_rows = local_pair && per_lane <= 4 && n_splits == 1 && n_tokens >= VT_TOKENS && (v_tiled || !write_kv);
    constexpr int MANY = 4;
    int grid = many_rows ? ceil_div(rows, QK_WAVES * MANY) : ceil_div(rows, QK_WAVES);
    size_t lds = local_pair ? 0 : (size_t)QK_WAVES * d * sizeof(float);
#define LAUNCH_N(TI, TO, N, LP)                                                                 \
    qk_norm_rope_append_kernel<TI, TO, N, LP><<<grid, EW_BLOCK, lds, stream>>>(                 \
        (const TI*)qkv, ld, n_tokens, hq, hkv, d, q_gain, k_gain, eps, cos_t, sin_t, rot,       \
        (TO*)q_out, (TO*)kcache, (TO*)vcache, block_table, bt_width, token_seq, token_pos,      \
        page_size, write_kv, n_splits, split_stride, rows_per_token, pairing, first_row)
#define LAUNCH_ROWS(TI, TO, N)                                                                  \
    qk_norm_rope_rows_kernel<TI, TO, N, MANY><<<grid, EW_BLOCK, 0, stream>>>(                   \
        (const TI*)qkv, ld, n_tokens, hq, hkv, d, q_gain, k_gain, eps, rot ? cos_t : nullptr,   \
        rot ? sin_t : nullptr, (TO*)q_out, (TO*)kcache, block_table, bt_width, token_seq,       \
        token_pos, page_size, rows_per_token, first_row)
#define LAUNCH(TI, TO)                                                                          \
    {                                                                                           \
        if (many_rows) { if (per_lane == 2) LAUNCH_ROWS(TI, TO, 2); else LAUNCH_ROWS(TI, TO, 4); } \
        else if (per_lane == 1) LAUNCH_N(TI, TO, 1, false);                                     \
        else if (per_lane == 2) { if (local_pair) LAUNCH_N(TI, TO, 2, true); else LAUNCH_N(TI, TO, 2, false); } \
        else if (per_lane == 4) { if (local_pair) LAUNCH_N(TI, TO, 4, true); else LAUNCH_N(TI, TO, 4, false); } \
        else { if (local_pair) LAUNCH_N(TI, TO, 8, true); else LAUNCH_N(TI, TO, 8, false); }    \
        if (v_tiled) {                                                                          \
            dim3 vgrid(ceil_div(n_tokens, VT_TOKENS), hkv, ceil_div(d, VT_VALUES));             \
            v_append_tile_kernel<TI, TO><<<vgrid, EW_BLOCK, 0, stream>>>(                       \
                (const TI*)qkv, ld, n_tokens, (hq + hkv) * d, hkv, d, (TO*)vcache, block_table, \
                bt_width, token_seq, token_pos, page_size);                                     \
        }                                                                                       \
    }
    if (in_dtype == ROCML_F32 && out_dtype == ROCML_F32) LAUNCH(float, float)
    else if (in_dtype == ROCML_F32 && out_dtype == ROCML_BF16) LAUNCH(float, bf16_t)
    else if (in_dtype == ROCML_BF16 && out_dtype == ROCML_BF16) LAUNCH(bf16_t, bf16_t)
    else return rocml_fail("qk_norm_rope_append: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
#undef LAUNCH
#undef LAUNCH_N
#undef LAUNCH_ROWS
    ROCML_CHECK_LAUNCH("qk_norm_rope_append");
    return 0;
}

// ---- residual add ----------------------------------------------------------------
// x += y  (rocml-kernels/kernels/elementwise.hip:7-12); parts without a fused epilogue use it.
template <typename T>
__global__ void add_into_kernel(float* __restrict__ x, const T* __restrict__ y, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx < total) x[idx] += Elem<T>::load(y + idx);
}

ROCML_EXPORT int rocml_add_into(float* x, const void* y, int y_dtype, long long total,
                                hipStream_t stream) {
    ROCML_REQUIRE(total >= 0, "add_into: negative size");
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (y_dtype == ROCML_F32) add_into_kernel<float><<<grid, EW_BLOCK, 0, stream>>>(x, (const float*)y, total);
    else if (y_dtype == ROCML_BF16) add_into_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>(x, (const bf16_t*)y, total);
    else return rocml_fail("add_into: unknown dtype code %d", y_dtype);
    ROCML_CHECK_LAUNCH("add_into");
    return 0;
}
