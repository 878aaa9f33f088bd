// bfloat16 attention over the paged cache on the gfx950 matrix cores.
//
// Cache layout (page_size = 64): keys [page, Hkv, 64, D], values transposed inside a page
// [page, Hkv, D, 64].  With this layout both products read 8 or 4 consecutive elements per
// lane: S^T = K * Q^T takes K rows along D, O^T = V^T * P^T takes V^T rows along the keys.
// Both kernels compute the transposed products so that one lane owns one query column: the
// running maximum, the sum and the rescaling of the output are lane-local and P^T is already
// the MFMA operand for the second product (no shuffles, no LDS round trip for P).
//
// The algebra is the reference's online softmax (rocml-kernels/kernels/attn_decode.hip:151-170,
// 227-254; attn_prefill_flash_impl.h:46-159): per query m' = max(m, s), acc and l scaled by
// e^(m - m'), splits merged by log-sum-exp in split order.  Scores are scaled after the dot
// product; exponentials are base 2 with log2(e) folded into the scale.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int AM_PAGE = 64;
constexpr int AM_THREADS = 256;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) { return f32x2_to_bf16x2(a, b); }

// Lane l and lane l ^ 32 combined (v_permlane32_swap: one VALU instruction instead of a trip
// through the LDS crossbar).  After the swap the first word holds the lower half's values in
// both halves of the wave and the second word the upper half's.
__device__ __forceinline__ float max_across_halves(float v) {
    typedef __attribute__((ext_vector_type(2))) unsigned u32x2_;
    u32x2_ r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_across_halves(float v) {
    typedef __attribute__((ext_vector_type(2))) unsigned u32x2_;
    u32x2_ r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- decode: one query token per sequence ----------------------------------------------------
// What the fused decode kernel reads in place of finished q rows and an appended cache row: the
// output of the q/k/v projection in 32-bit (or its split-K partial sums, [splits][tokens][ld]),
// the gains of the per-head norm (null: no norm) and the rotation tables (null: no rotation;
// else the whole head is rotated, pairs (e, e + D/2)).
// row_ssq (null: none): the projection's operand was bfloat16(x * gain) of a norm whose scale is
// still to come; row_ssq[token][row_parts] are sums of squares of x, and every sum of the
// projection is multiplied by 1 / sqrt(sum of the token's parts * row_inv_width + row_eps) first.
struct DecodeProj {
    const float* qkv; int ld; int n_splits; long long split_stride;
    const float* q_gain; const float* k_gain; float eps;
    const float* cos_t; const float* sin_t; int write_kv;
    const float* row_ssq; int row_parts; float row_eps; float row_inv_width;
};

// grid (n_splits, Hkv, tokens), 4 or 8 waves; the block's pages are cut into 32-key pieces that the
// waves take in turn; all query heads of the kv head ride in the 16 columns of the MFMA.
//
// FUSED: the kernel takes the projection's output instead of q and a finished cache: every block
// norms and rotates the q heads of its kv head itself and lays them out as the MFMA operand; the
// block whose split holds the sequence's last page also norms and rotates the new key, writes it
// and the new value into the cache and multiplies them as one more piece, from LDS: the loads
// from the cache may or may not see a row that is written in the same launch, so the cached
// keys end before it.  A page belongs to one split, so no other block reads that row.
// WAVES: 4, or 8 for launches of at most one block a CU whose blocks have many pieces: a wave
// then has half as many, and the pieces of a block travel in half as many trips.
template <int D, bool FUSED, int AHEAD, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
attn_decode_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                        bf16_t* kcache, bf16_t* vcache,
                        const int* __restrict__ block_table, int bt_width,
                        const int* __restrict__ token_seq, const int* __restrict__ token_pos, int hq,
                        int hkv, float scale_log2e, int window, int n_splits,
                        float* __restrict__ part_o, float* __restrict__ part_ml, DecodeProj pj) {
    constexpr int KD = D / 32;      // MFMA steps along D for the scores
    constexpr int DT = D / 16;      // 16-row tiles of the output
    constexpr int THREADS = 64 * WAVES;
    extern __shared__ float sm_o[];                 // [WAVES][group][D + 4]
    __shared__ float sm_m[WAVES][16], sm_l[WAVES][16];
    int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int g = lane >> 4, col = lane & 15;
    int group = hq / hkv;
    // (token_seq null: token t is the one token of the step's sequence t)
    const int* pages = block_table + (size_t)(token_seq ? token_seq[t] : t) * bt_width;
    // Without a window a split's pages are split, split + n_splits, ... whatever the length: the
    // first four are looked up together with the position, a trip to memory earlier.
    int early[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) early[i] = pages[split + i * n_splits < bt_width ? split + i * n_splits : 0];
    int len = token_pos[t] + 1;
    int lo = window > 0 ? max(0, len - window) : 0;
    int first_page = lo / AM_PAGE;
    int n_pages = (len + AM_PAGE - 1) / AM_PAGE - first_page;
    // split s takes pages s, s + n_splits, ...: the splits of a sequence, which run side by side,
    // then read neighbouring pages at any one time instead of n_splits distant ranges
    int my_pages = split < n_pages ? (n_pages - split + n_splits - 1) / n_splits : 0;
    int n_pieces = my_pages * 2;

    const bf16_t* knew_lds = nullptr;
    const bf16_t* vnew_lds = nullptr;
    // Row r of score tile u is key 8 (r / 4) + 4u + r % 4 of a piece: then the 8 keys whose
    // probabilities a lane holds after the softmax (rows 4g .. 4g+3 of both tiles) are the
    // consecutive keys 8g .. 8g+7, and its values for them are one 16-byte load.
    // AHEAD = 2: two pieces are on their way at a time.  A block of a small batch has a piece or
    // two per wave, and their trips to memory then overlap; long loops gain nothing from it and
    // lose a block per CU to the registers.
    uint4 kbuf[AHEAD][2][KD], vbuf[AHEAD][DT];
    auto request_piece = [&](int piece, uint4 (&kreg)[2][KD], uint4 (&vreg)[DT]) {
        // (the page index is the same for all lanes: a scalar load)
        int round = __builtin_amdgcn_readfirstlane(piece >> 1), half = piece & 1;
        int phys;
        if (window == 0 && round < 4)
            phys = round == 0 ? early[0] : round == 1 ? early[1] : round == 2 ? early[2] : early[3];
        else
            phys = pages[first_page + split + round * n_splits];
        const bf16_t* kbase = kcache + (((size_t)phys * hkv + kvh) * AM_PAGE + half * 32) * D;
        const bf16_t* vbase = vcache + ((size_t)phys * hkv + kvh) * D * AM_PAGE + half * 32;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const bf16_t* krow = kbase + (size_t)(8 * (col >> 2) + 4 * u + (col & 3)) * D + g * 8;
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) kreg[u][kd] = *(const uint4*)(krow + kd * 32);
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            vreg[dt] = *(const uint4*)(vbase + (size_t)(dt * 16 + col) * AM_PAGE + g * 8);
    };
    // The wave's first pieces are requested before the queries: their keys and values travel
    // together with them.
    if (wave < n_pieces) request_piece(wave, kbuf[0], vbuf[0]);
    if (AHEAD == 2 && wave + WAVES < n_pieces) request_piece(wave + WAVES, kbuf[AHEAD - 1], vbuf[AHEAD - 1]);
    // Q^T operand: column = head of the group (zero beyond it), 8 values of D per lane and step.
    bf16x8_t qf[KD];
    bool owner = false;      // this block appends the new key and value
    int new_pos = len - 1;
    if constexpr (!FUSED) {
        bool ok = col < group;
        const bf16_t* qrow = q + ((size_t)t * hq + kvh * group + (ok ? col : 0)) * D + g * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            uint4 v = *(const uint4*)(qrow + kd * 32);
            v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
            qf[kd] = __builtin_bit_cast(bf16x8_t, v);
        }
    } else {
        // Rows of the projection this block turns into operands: the q heads of its kv head and,
        // in the block whose split holds the sequence's last page, the new key and value.  A wave
        // takes a row at a time, a lane the values lane, lane + 64, ...; two rows per wave are
        // loaded together, so a group of four heads with key and value is one trip to memory.
        constexpr int J = D / 64;
        __shared__ float sm_f[WAVES][2][D];                        // a row before its rotation
        __shared__ __attribute__((aligned(16))) bf16_t sm_q[16 * D];        // [head of the group][D]
        __shared__ __attribute__((aligned(16))) bf16_t sm_knew[D];
        __shared__ __attribute__((aligned(16))) bf16_t sm_vnew[D];
        int last_lpage = new_pos / AM_PAGE;
        owner = pj.write_kv && (last_lpage - first_page) % n_splits == split;
        int n_rows = group + (owner ? 2 : 0);       // q heads, then key, then value
        const float* tok = pj.qkv + (size_t)t * pj.ld;
        float row_scale = 1.0f;
        if (pj.row_ssq) {           // (every wave forms the same number in the same order)
            float ss = 0.f;
            const float* row = pj.row_ssq + (size_t)t * pj.row_parts;
            if ((pj.row_parts & 3) == 0) {
                for (int c = lane; c < pj.row_parts / 4; c += 64) {
                    float4 v = ((const float4*)row)[c];
                    ss += (v.x + v.y) + (v.z + v.w);
                }
            } else {
                for (int p = lane; p < pj.row_parts; p += 64) ss += row[p];
            }
            row_scale = 1.0f / sqrtf(wave_sum(ss) * pj.row_inv_width + pj.row_eps);
        }
        for (int base = 0; base < n_rows; base += 2 * WAVES) {
            int r[2];
            const float* src[2];
            float raw[2][J][4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                r[i] = base + i * WAVES + wave;
                int prow = r[i] < group ? kvh * group + r[i] : (r[i] == group ? hq + kvh : hq + hkv + kvh);
                src[i] = tok + (size_t)(r[i] < n_rows ? prow : 0) * D + lane;
#pragma unroll
                for (int j = 0; j < J; ++j)
#pragma unroll
                    for (int sp = 0; sp < 4; ++sp)
                        raw[i][j][sp] = src[i][j * 64 + (sp < pj.n_splits ? sp * pj.split_stride : 0)];
            }
            float val[2][J];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                // split-K partial sums of the projection, added in split order
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    float a = raw[i][j][0];
#pragma unroll
                    for (int sp = 1; sp < 4; ++sp)
                        if (sp < pj.n_splits) a += raw[i][j][sp];
                    for (int sp = 4; sp < pj.n_splits; ++sp) a += src[i][j * 64 + sp * pj.split_stride];
                    val[i][j] = a * row_scale;
                }
                const float* gain = r[i] < group ? pj.q_gain : (r[i] == group ? pj.k_gain : nullptr);
                if (gain) {
                    float ss = 0.f;
#pragma unroll
                    for (int j = 0; j < J; ++j) ss = fmaf(val[i][j], val[i][j], ss);
                    float inv = 1.0f / sqrtf(wave_sum(ss) / (float)D + pj.eps);
#pragma unroll
                    for (int j = 0; j < J; ++j) val[i][j] = val[i][j] * inv * gain[lane + j * 64];
                }
#pragma unroll
                for (int j = 0; j < J; ++j) sm_f[wave][i][lane + j * 64] = val[i][j];
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (r[i] >= n_rows) continue;
                bool rotate = pj.cos_t != nullptr && r[i] <= group;
                const float* c = pj.cos_t + (size_t)t * (D / 2);
                const float* sn = pj.sin_t + (size_t)t * (D / 2);
                bf16_t* dst = r[i] < group ? sm_q + r[i] * D : (r[i] == group ? sm_knew : sm_vnew);
                int phys = pages[last_lpage], in_page = new_pos % AM_PAGE;
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    int e = lane + j * 64;
                    float x = val[i][j];
                    if (rotate) {
                        if (e < D / 2) x = x * c[e] - sm_f[wave][i][e + D / 2] * sn[e];
                        else x = sm_f[wave][i][e - D / 2] * sn[e - D / 2] + x * c[e - D / 2];
                    }
                    bf16_t xb = f32_to_bf16(x);
                    dst[e] = xb;
                    if (r[i] == group && phys >= 0)
                        kcache[(((size_t)phys * hkv + kvh) * AM_PAGE + in_page) * D + e] = xb;
                    if (r[i] == group + 1 && phys >= 0)
                        vcache[(((size_t)phys * hkv + kvh) * D + e) * AM_PAGE + in_page] = xb;
                }
            }
            __syncthreads();
        }
        {
            bool ok = col < group;
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                uint4 v = *(const uint4*)(sm_q + (ok ? col : 0) * D + kd * 32 + g * 8);
                v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
                qf[kd] = __builtin_bit_cast(bf16x8_t, v);
            }
        }
        knew_lds = sm_knew;
        vnew_lds = sm_vnew;
    }
    float m = -INFINITY, l = 0.f;
    f32x4_t o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // All loads of a piece go out before anything is computed, the values too: a block has
    // few pieces, and keys, softmax, values one after the other would be two trips to memory
    // per piece where one will do.
    // keys [key0, key0 + 32) of which those in [from, to) count
    auto multiply_piece = [&](int key0, int from, int to, const uint4 (&kreg)[2][KD], const uint4 (&vreg)[DT]) {
        __builtin_amdgcn_sched_barrier(0);
        // scores of 2 x 16 keys: element i of s[u] is key 8g + 4u + i, column = head.
        f32x4_t s[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            s[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kd = 0; kd < KD; ++kd)
                s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kreg[u][kd]), qf[kd], s[u], 0, 0, 0);
        }
        float mx = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int key = key0 + g * 8 + u * 4 + i;
                float v = (key >= from && key < to) ? s[u][i] * scale_log2e : -INFINITY;
                s[u][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float m_new = fmaxf(m, mx);
        float m_use = m_new == -INFINITY ? 0.f : m_new;
        float corr = fast_exp2(m - m_use);
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[u][i] = fast_exp2(s[u][i] - m_use);
                sum += s[u][i];
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l = l * corr + sum;
        m = m_new;
        // P^T operand: slots 0..7 = keys 8g .. 8g+7.
        uint4 pv = make_uint4(pack_bf16x2(s[0][0], s[0][1]), pack_bf16x2(s[0][2], s[0][3]),
                              pack_bf16x2(s[1][0], s[1][1]), pack_bf16x2(s[1][2], s[1][3]));
        bf16x8_t pf = __builtin_bit_cast(bf16x8_t, pv);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            o[dt] = o[dt] * corr;
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vreg[dt]), pf, o[dt], 0, 0, 0);
        }
    };
    // (FUSED: the new key is not yet in the cache where a block reads it; it comes last, from LDS)
    int cached = (FUSED && owner) ? new_pos : len;
    auto first_key = [&](int piece) { return (first_page + split + (piece >> 1) * n_splits) * AM_PAGE + (piece & 1) * 32; };
    for (int piece = wave; piece < n_pieces; piece += WAVES * AHEAD) {
        multiply_piece(first_key(piece), lo, cached, kbuf[0], vbuf[0]);
        if (piece + WAVES * AHEAD < n_pieces) request_piece(piece + WAVES * AHEAD, kbuf[0], vbuf[0]);
        if (AHEAD == 2 && piece + WAVES < n_pieces) {
            multiply_piece(first_key(piece + WAVES), lo, cached, kbuf[AHEAD - 1], vbuf[AHEAD - 1]);
            if (piece + 3 * WAVES < n_pieces) request_piece(piece + 3 * WAVES, kbuf[AHEAD - 1], vbuf[AHEAD - 1]);
        }
    }
    if constexpr (FUSED) {
        // The step's own key and value as a piece of their own, row 0 of score tile 0, in the
        // wave whose turn would be next.
        if (owner && wave == n_pieces % WAVES) {
            bool krow = col == 0, vrow = g == 0;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    uint4 v = *(const uint4*)(knew_lds + kd * 32 + g * 8);
                    bool take = krow && u == 0;
                    kbuf[0][u][kd] = make_uint4(take ? v.x : 0u, take ? v.y : 0u, take ? v.z : 0u, take ? v.w : 0u);
                }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                vbuf[0][dt] = make_uint4(vrow ? (uint32_t)vnew_lds[dt * 16 + col] : 0u, 0u, 0u, 0u);
            multiply_piece(new_pos, new_pos, new_pos + 1, kbuf[0], vbuf[0]);
        }
    }
    // merge the waves in wave order; element i of o[dt] is d = 16 dt + 4g + i, column = head.
    if (col < group) {
        float* mine = sm_o + ((size_t)wave * group + col) * (D + 4);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[dt * 16 + g * 4 + i] = o[dt][i];
    }
    if (g == 0) {
        sm_m[wave][col] = m;
        sm_l[wave][col] = l;
    }
    __syncthreads();
    for (int idx = tid; idx < group * D; idx += THREADS) {
        int head = idx / D, d = idx - head * D;
        float mm = sm_m[0][head];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) mm = fmaxf(mm, sm_m[w][head]);
        float ll = 0.f, acc = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            float wgt = sm_m[w][head] == -INFINITY ? 0.f : fast_exp2(sm_m[w][head] - mm);
            ll += sm_l[w][head] * wgt;
            acc += sm_o[((size_t)w * group + head) * (D + 4) + d] * wgt;
        }
        int h = kvh * group + head;
        if (n_splits == 1) {
            out[((size_t)t * hq + h) * D + d] = f32_to_bf16(acc / ll);
        } else {
            size_t slot = ((size_t)t * hq + h) * n_splits + split;
            part_o[slot * D + d] = acc;
            if (d == 0) {
                part_ml[slot * 2] = mm;
                part_ml[slot * 2 + 1] = ll;
            }
        }
    }
}

// Log-sum-exp merge of the splits in split order (rocml-kernels/kernels/attn_decode.hip:219-255).
template <int D>
__global__ void attn_decode_reduce_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          bf16_t* __restrict__ out, int n_splits) {
    // At most 64 splits: lane s of every wave fetches split s's maximum and sum, so the loads
    // go out together; the weights then sit in LDS for the sum over splits.  The partial
    // outputs of the first eight splits are requested before the weights are formed: the
    // kernel is one trip to memory for them.  The block has at least D threads.
    __shared__ float wgt[64];
    int row = blockIdx.x;     // token * Hq + head
    const float* ml = part_ml + (size_t)row * n_splits * 2;
    const float* po = part_o + (size_t)row * n_splits * D;
    int lane = threadIdx.x & 63;
    int d = threadIdx.x < D ? threadIdx.x : 0;
    bool has = lane < n_splits;
    float ms = has ? ml[lane * 2] : -INFINITY;
    float ls = has ? ml[lane * 2 + 1] : 0.f;
    float first[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) first[s] = po[(size_t)min(s, n_splits - 1) * D + d];
    float mm = wave_max(ms);
    float w = ms == -INFINITY ? 0.f : fast_exp2(ms - mm);
    if (threadIdx.x < 64) wgt[lane] = w;
    float inv_l = 1.0f / wave_sum(ls * w);          // every wave computes the same sum
    __syncthreads();
    // (splits beyond the last have weight zero, and their loads are aimed at the last split's
    // finite values: no branches)
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) acc += first[s] * wgt[s];
    for (int s0 = 8; s0 < n_splits; s0 += 8) {
        float more[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) more[s] = po[(size_t)min(s0 + s, n_splits - 1) * D + d];
#pragma unroll
        for (int s = 0; s < 8; ++s) acc += more[s] * wgt[s0 + s];
    }
    if (threadIdx.x < D) out[(size_t)row * D + d] = f32_to_bf16(acc * inv_l);
}

// ---- prefill: many query tokens per sequence --------------------------------------------------
// grid: query tiles of AM_QTILE rows over all sequences x Hq, 4 waves of 32 query rows.  Pages of
// keys and values go through LDS once per block; every wave multiplies its 32 queries with them.
constexpr int AM_ROUND = 256;                           // blocks that start together: one per CU
constexpr int AM_QTILE = 128;                           // query rows of a block: 32 per wave
constexpr float AM_LAZY_MAX = 8.0f;                     // how far a row's maximum may run ahead of its exponents' reference

template <int D>
struct PrefillLds {
    static constexpr int K_ROW = D + 8;                 // bf16 per key row (16 bytes of padding)
    static constexpr int V_ROW = AM_PAGE + 8;           // bf16 per value row (16 bytes of padding)
    static constexpr int BYTES = (AM_PAGE * K_ROW + D * V_ROW) * 2;
};

// QPREP: the queries come as the step's q/k/v projection (32-bit, complete sums) and are
// prepared here, per-head norm, rotation of the whole head with pairs (e, e + D/2) and rounding,
// as the norm-and-rotation kernel would have prepared them; that kernel then only appends keys and
// values, and the queries are neither written nor read as bfloat16 in between.
struct PrefillProj {
    const float* qkv; int ld;                           // [T, ld]: a token's q heads first
    const float* q_gain; float eps;                     // null: no norm
    const float* cos_t; const float* sin_t;             // [T, D/2], null: no rotation
};

template <int D, bool QPREP>
__global__ void __launch_bounds__(AM_THREADS, D <= 128 ? 2 : 1)
attn_prefill_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                         const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                         const int* __restrict__ block_table, int bt_width,
                         const int* __restrict__ cu_seqlens, int n_seqs,
                         const int* __restrict__ token_pos, int hq, int hkv, float scale_log2e,
                         int window, PrefillProj pj) {
    using L = PrefillLds<D>;
    constexpr int KK = D / 16;      // MFMA steps along D for the scores
    constexpr int DT = D / 32;      // 32-row tiles of the output
    extern __shared__ uint4 am_smem[];
    bf16_t* sk = (bf16_t*)am_smem;
    bf16_t* sv = sk + AM_PAGE * L::K_ROW;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int h2 = lane >> 5, col = lane & 31;
    // Which tile and head.  The last tile of a sequence sees the most keys, the first the fewest.
    // Blocks are numbered so that (a) heavy tiles come first, all heads of a tile side by side,
    // and (b) every other round of AM_ROUND blocks runs backwards: the hardware hands block
    // numbers out in order, a CU that got the r-th heaviest block of a round gets the r-th
    // lightest of the next, and when all blocks are resident at once (a 2048-token prompt) the
    // CUs carry equal sums instead of twice the heaviest and twice the lightest.
    int n_blocks = gridDim.x, total_tiles = n_blocks / hq;
    int round0 = (blockIdx.x / AM_ROUND) * AM_ROUND, in_round = blockIdx.x - round0;
    int round_size = min(AM_ROUND, n_blocks - round0);
    int s = round0 + (((blockIdx.x / AM_ROUND) & 1) ? round_size - 1 - in_round : in_round);
    int h = s % hq, kvh = h / (hq / hkv);
    int tile = total_tiles - 1 - s / hq, b = 0, tok0 = 0, n_new = 0;
    for (; b < n_seqs; ++b) {
        tok0 = cu_seqlens[b];
        n_new = cu_seqlens[b + 1] - tok0;
        int tiles = (n_new + AM_QTILE - 1) / AM_QTILE;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (b >= n_seqs) return;
    const int* pages = block_table + (size_t)b * bt_width;
    int pos0 = token_pos[tok0];                        // position of the sequence's first new token
    int row_lo = tile * AM_QTILE, row_hi = min(n_new, row_lo + AM_QTILE) - 1;     // block's query rows
    int w_lo = row_lo + wave * 32, w_hi = min(n_new - 1, w_lo + 31);    // wave's query rows
    bool wave_active = w_lo < n_new;
    int my_row = w_lo + col;
    bool row_ok = my_row < n_new;
    int my_pos = pos0 + my_row;
    int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
    int blk_first_key = window > 0 ? max(0, pos0 + row_lo - window + 1) : 0;
    int blk_last_key = pos0 + row_hi;
    int wave_first_key = window > 0 ? max(0, pos0 + w_lo - window + 1) : 0;
    int wave_last_key = pos0 + w_hi;

    // Q^T operand: column = query row, 8 values of D per lane and step.
    bf16x8_t qf[KK];
    if constexpr (QPREP) {
        // this lane's 8 values of every 16 of its row; the other 8 are in the lane 32 away
        int t = tok0 + (row_ok ? my_row : 0);
        const float* qrow = pj.qkv + (size_t)t * pj.ld + (size_t)h * D + h2 * 8;
        float qv[KK][8];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            float4 lo = *(const float4*)(qrow + kk * 16), hi = *(const float4*)(qrow + kk * 16 + 4);
            qv[kk][0] = lo.x; qv[kk][1] = lo.y; qv[kk][2] = lo.z; qv[kk][3] = lo.w;
            qv[kk][4] = hi.x; qv[kk][5] = hi.y; qv[kk][6] = hi.z; qv[kk][7] = hi.w;
        }
        if (pj.q_gain) {
            float ss = 0.f;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                for (int i = 0; i < 8; ++i) ss = fmaf(qv[kk][i], qv[kk][i], ss);
            ss += __shfl_xor(ss, 32, 64);
            float inv = 1.0f / sqrtf(ss / (float)D + pj.eps);
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const float* g = pj.q_gain + kk * 16 + h2 * 8;
                float4 g0 = *(const float4*)g, g1 = *(const float4*)(g + 4);
                qv[kk][0] *= inv * g0.x; qv[kk][1] *= inv * g0.y; qv[kk][2] *= inv * g0.z; qv[kk][3] *= inv * g0.w;
                qv[kk][4] *= inv * g1.x; qv[kk][5] *= inv * g1.y; qv[kk][6] *= inv * g1.z; qv[kk][7] *= inv * g1.w;
            }
        }
        if (pj.cos_t) {
            // value e of the first half of the head and value e + D/2 are a pair: steps kk and kk + KK/2
            const float* c = pj.cos_t + (size_t)t * (D / 2) + h2 * 8;
            const float* sn = pj.sin_t + (size_t)t * (D / 2) + h2 * 8;
#pragma unroll
            for (int kk = 0; kk < KK / 2; ++kk) {
                float cs[8], si[8];
                *(float4*)cs = *(const float4*)(c + kk * 16); *(float4*)(cs + 4) = *(const float4*)(c + kk * 16 + 4);
                *(float4*)si = *(const float4*)(sn + kk * 16); *(float4*)(si + 4) = *(const float4*)(sn + kk * 16 + 4);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float lo = qv[kk][i], hi = qv[kk + KK / 2][i];
                    qv[kk][i] = lo * cs[i] - hi * si[i];
                    qv[kk + KK / 2][i] = lo * si[i] + hi * cs[i];
                }
            }
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            uint4 v = make_uint4(pack_bf16x2(qv[kk][0], qv[kk][1]), pack_bf16x2(qv[kk][2], qv[kk][3]),
                                 pack_bf16x2(qv[kk][4], qv[kk][5]), pack_bf16x2(qv[kk][6], qv[kk][7]));
            v.x = row_ok ? v.x : 0u; v.y = row_ok ? v.y : 0u; v.z = row_ok ? v.z : 0u; v.w = row_ok ? v.w : 0u;
            qf[kk] = __builtin_bit_cast(bf16x8_t, v);
        }
    } else {
        const bf16_t* qrow = q + ((size_t)(tok0 + (row_ok ? my_row : 0)) * hq + h) * D + h2 * 8;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            uint4 v = *(const uint4*)(qrow + kk * 16);
            v.x = row_ok ? v.x : 0u; v.y = row_ok ? v.y : 0u; v.z = row_ok ? v.z : 0u; v.w = row_ok ? v.w : 0u;
            qf[kk] = __builtin_bit_cast(bf16x8_t, v);
        }
    }
    float m = -INFINITY, l = 0.f;
    f32x16_t o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[i][e] = 0.f;

    // A page's keys and values wait in registers while the page before it is multiplied out of
    // LDS: the loads of page p + 1 are issued right after page p has been written to LDS.
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    constexpr int K_PIECES = AM_PAGE * D / 8 / AM_THREADS, V_PIECES = D * AM_PAGE / 8 / AM_THREADS;
    u32x4 kreg[K_PIECES], vreg[V_PIECES];
    int first_page = blk_first_key / AM_PAGE, last_page = blk_last_key / AM_PAGE;
#define AM_LOAD_PAGE(lp_)                                                                         \
    {                                                                                             \
        int phys_ = pages[lp_];                                                                   \
        const u32x4* gk_ = (const u32x4*)(kcache + ((size_t)phys_ * hkv + kvh) * AM_PAGE * D);    \
        const u32x4* gv_ = (const u32x4*)(vcache + ((size_t)phys_ * hkv + kvh) * D * AM_PAGE);    \
        _Pragma("unroll") for (int i = 0; i < K_PIECES; ++i) kreg[i] = gk_[tid + i * AM_THREADS]; \
        _Pragma("unroll") for (int i = 0; i < V_PIECES; ++i) vreg[i] = gv_[tid + i * AM_THREADS]; \
    }
    // the wave's rows see every key of a 32-key piece when the piece lies at or below the first
    // row's position and at or above the last row's window start; only then masking is skipped
    int wave_min_pos = pos0 + w_lo;
    int wave_max_lo = window > 0 ? max(0, pos0 + w_hi - window + 1) : 0;
    bool wave_full = w_hi - w_lo == 31;
    AM_LOAD_PAGE(first_page)
    for (int lpage = first_page; lpage <= last_page; ++lpage) {
        __syncthreads();                                // the previous page has been consumed
#pragma unroll
        for (int i = 0; i < K_PIECES; ++i) {
            int piece = tid + i * AM_THREADS;
            int key = piece / (D / 8), dc = piece % (D / 8);
            *(u32x4*)(sk + key * L::K_ROW + dc * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < V_PIECES; ++i) {
            int piece = tid + i * AM_THREADS;
            // Within 16 keys the four groups of 4 stand in the order 0, 2, 1, 3: the second product
            // wants keys {4h .. 4h+3, 8+4h .. 8+4h+3} per lane (the order the scores come in), and
            // so finds them side by side, one 16-byte read.
            int d = piece / 8, kc = piece % 8;
            uint2* dst = (uint2*)(sv + d * L::V_ROW + (kc >> 1) * 16 + (kc & 1) * 4);
            dst[0] = make_uint2(vreg[i][0], vreg[i][1]);
            dst[2] = make_uint2(vreg[i][2], vreg[i][3]);
        }
        __syncthreads();
        if (lpage < last_page) AM_LOAD_PAGE(lpage + 1)
        if (!wave_active) continue;
        // The scores of both 32-key halves are started before either is finished: the softmax of
        // the first half (vector ALU) then runs while the matrix core still multiplies the second,
        // and the softmax of the second while the first half's values are multiplied.
        // S^T: element e of s is key 8(e/4) + 4 h2 + e%4, column = query row.
        int page_key0 = lpage * AM_PAGE;
        bool live[2];
        f32x16_t sc[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            int key0 = page_key0 + half * 32;
            live[half] = !(key0 > wave_last_key || key0 + 31 < wave_first_key);   // wave-uniform
            if (!live[half]) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) sc[half][e] = 0.f;
            const bf16_t* krow = sk + (half * 32 + col) * L::K_ROW + h2 * 8;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                bf16x8_t kf = __builtin_bit_cast(bf16x8_t, *(const uint4*)(krow + kk * 16));
                sc[half] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], sc[half], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            if (!live[half]) continue;
            int key0 = page_key0 + half * 32;
            f32x16_t& s = sc[half];
            bool need_mask = !wave_full || key0 + 31 > wave_min_pos || key0 < wave_max_lo;   // wave-uniform
            if (need_mask) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int key = key0 + 8 * (e >> 2) + 4 * h2 + (e & 3);
                    s[e] = (row_ok && key <= my_pos && key >= my_lo) ? s[e] : -INFINITY;
                }
            }
            float mx = s[0];
#pragma unroll
            for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s[e]);
            mx = max_across_halves(mx) * scale_log2e;       // the scale is positive
            // The exponents' reference m follows a row's maximum only when that has grown by more
            // than AM_LAZY_MAX (powers of two): any reference gives the same quotient at the end,
            // the probabilities stay below 2^AM_LAZY_MAX, which bfloat16 and the 32-bit sums hold
            // with room to spare, and the sums and outputs so far have to be rescaled (64 products
            // a lane) only for the first pieces of a row instead of whenever one of a wave's 32
            // rows meets a new maximum, which with a thousand keys behind it is still every other piece.
            if (__builtin_amdgcn_ballot_w64(mx > m + AM_LAZY_MAX)) {
                float m_new = fmaxf(m, mx);
                float corr = fast_exp2(m - (m_new == -INFINITY ? 0.f : m_new));
                l *= corr;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[dt][e] *= corr;
                m = m_new;
            }
            float m_use = m == -INFINITY ? 0.f : m;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                s[e] = fast_exp2(fmaf(s[e], scale_log2e, -m_use));
                sum += s[e];
            }
            sum = sum_across_halves(sum);
            l += sum;
            // P^T operands: MFMA u takes elements 8u..8u+7 = keys 16u + {4 h2 .. +3, 8 + 4 h2 .. +3}.
            bf16x8_t pf[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
                pf[u] = __builtin_bit_cast(bf16x8_t, make_uint4(
                    pack_bf16x2(s[8 * u + 0], s[8 * u + 1]), pack_bf16x2(s[8 * u + 2], s[8 * u + 3]),
                    pack_bf16x2(s[8 * u + 4], s[8 * u + 5]), pack_bf16x2(s[8 * u + 6], s[8 * u + 7])));
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16_t* vrow = sv + (dt * 32 + col) * L::V_ROW + half * 32 + 16 * u + 8 * h2;
                    bf16x8_t vf = __builtin_bit_cast(bf16x8_t, *(const uint4*)vrow);
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[u], o[dt], 0, 0, 0);
                }
            }
        }
    }
#undef AM_LOAD_PAGE
    if (!row_ok) return;
    float inv = 1.0f / l;
    bf16_t* orow = out + ((size_t)(tok0 + my_row) * hq + h) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            int d = dt * 32 + 8 * e4 + 4 * h2;
            uint2 v = make_uint2(pack_bf16x2(o[dt][4 * e4] * inv, o[dt][4 * e4 + 1] * inv),
                                 pack_bf16x2(o[dt][4 * e4 + 2] * inv, o[dt][4 * e4 + 3] * inv));
            *(uint2*)(orow + d) = v;
        }
}
