// Sampling on the device, one 1024-thread block per sequence, in the order of the reference's
// host sampler (rocml/src/sample.rs:90-166): repeat penalty over recent history, greedy if the
// temperature is not positive (first maximum wins, :172-182), else scale by 1/temperature,
// keep the top k, softmax, keep the smallest set of most probable tokens whose mass reaches
// top_p, draw with the caller's uniform number.
#include "common.h"
#include "sampling.h"
#include <mutex>

ROCML_LAST_ERROR_FN(sampling)

constexpr int SB = 256;
constexpr int SAMPLE_THREADS = 1024;        // the sampling kernel reads a row dozens of times: a big block, 16 bytes per load
constexpr int SAMPLE_MAX_VOCAB = 1 << 20;   // the draw keeps one sum per 256 values in LDS

struct ArgMax { float v; int i; };

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
    // larger value wins; on a tie the lower index wins ("first maximum").
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

template <int THREADS = SB>
__device__ ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        ArgMax o;
        o.v = __shfl_xor(a.v, off, 64);
        o.i = __shfl_xor(a.i, off, 64);
        a = better(a, o);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = a;
    __syncthreads();
    ArgMax r = scratch[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) r = better(r, scratch[w]);
    return r;
}

template <int THREADS = SB>
__device__ float block_sum_f(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) r += scratch[w];
    return r;
}

template <int THREADS = SB>
__device__ int block_sum_i(int v, int* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = v;
    __syncthreads();
    int r = 0;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) r += scratch[w];
    return r;
}

// e^x for x <= 0 through the hardware's 2^x (v_exp_f32, about one unit in the last place): a
// sampling call takes the exponential of the whole vocabulary on one CU.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// Order-preserving map of a float to an unsigned key (larger float -> larger key).  The two
// zeros compare equal as numbers and so share one key: a tie between them goes by token id.
__device__ __forceinline__ uint32_t float_key(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Penalised logit of token i: a token among the last `window` history entries has a positive
// logit divided by the penalty and any other multiplied (rocml/src/sample.rs:188-202).  The
// reference applies the penalty once per occurrence; `hist` holds each recent token once per
// occurrence too, so the count is the same.
__device__ __forceinline__ float penalised(float v, int i, const int* hist, int n_hist, float penalty) {
    for (int j = 0; j < n_hist; ++j)
        if (hist[j] == i) v = v > 0.f ? v / penalty : v * penalty;
    return v;
}

// The largest of 256 bins whose sum from the top (itself included) reaches `need`, and the sum of
// the bins above it; bin 0 if the whole histogram falls short.  Called by the 64 lanes of one
// wave, each with four bins; the sums are integers, so the order of the additions is free.
template <typename T>
__device__ __forceinline__ void bin_from_top(const T* bins, T need, int lane, int* bin_out, T* above_out) {
    T mine = bins[4 * lane] + bins[4 * lane + 1] + bins[4 * lane + 2] + bins[4 * lane + 3];
    T suffix = mine;                                     // bins of this lane and of all higher lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        T o = __shfl_down(suffix, off, 64);
        if (lane + off < 64) suffix += o;
    }
    unsigned long long reach = __builtin_amdgcn_ballot_w64(suffix >= need);
    int owner = reach ? 63 - __builtin_clzll(reach) : -1;   // the highest lane from which the top still reaches
    if (owner < 0) {
        if (lane == 0) { *bin_out = 0; *above_out = suffix - bins[0]; }
        return;
    }
    if (lane == owner) {
        T above = suffix - mine;
        int bin = 4 * lane + 3;
        for (; bin > 4 * lane; --bin) {
            if (above + bins[bin] >= need) break;
            above += bins[bin];
        }
        *bin_out = bin;
        *above_out = above;
    }
}

// One pass over a row of `n_` floats by the whole block: BODY sees every index `i_` once with its
// value `v_`.  Loads go out in batches (four of 16 bytes where the row is aligned, else eight of
// 4 bytes) before any of them is used: a loop that waits for each load in turn spends its time on
// latency, and a sampling call makes a dozen passes.  `vec_ok_`: the row starts on 16 bytes.
#define SAMPLE_ROW_PASS(row_, n_, vec_ok_, i_, v_, ...)                                           \
    {                                                                                             \
        int nvec_ = (vec_ok_) ? (n_) / 4 : 0;                                                     \
        const float4* row4_ = (const float4*)(row_);                                              \
        for (int base_ = tid; base_ < nvec_; base_ += 4 * SB) {                                   \
            float4 ld_[4];                                                                        \
            _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) ld_[u_] = row4_[min(base_ + u_ * SB, nvec_ - 1)]; \
            _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) {                                    \
                if (base_ + u_ * SB < nvec_) {                                                    \
                    float e_[4] = {ld_[u_].x, ld_[u_].y, ld_[u_].z, ld_[u_].w};                   \
                    _Pragma("unroll") for (int c_ = 0; c_ < 4; ++c_) {                            \
                        int i_ = (base_ + u_ * SB) * 4 + c_;                                      \
                        float v_ = e_[c_];                                                        \
                        __VA_ARGS__                                                               \
                    }                                                                             \
                }                                                                                 \
            }                                                                                     \
        }                                                                                         \
        for (int base_ = nvec_ * 4 + tid; base_ < (n_); base_ += 8 * SB) {                        \
            float ld_[8];                                                                         \
            _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_) ld_[u_] = (row_)[min(base_ + u_ * SB, (n_) - 1)]; \
            _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_) {                                    \
                int i_ = base_ + u_ * SB;                                                         \
                if (i_ < (n_)) {                                                                  \
                    float v_ = ld_[u_];                                                           \
                    __VA_ARGS__                                                                   \
                }                                                                                 \
            }                                                                                     \
        }                                                                                         \
    }

// The same walk for a pass that rewrites the row: BODY sets `o_` from index `i_` and value `v_`,
// and the results go out 16 bytes at a time where both rows are aligned (single 4-byte stores of
// neighbouring lanes land 16 bytes apart and each touches a line of its own).
#define SAMPLE_ROW_MAP(in_, out_, n_, vec_ok_, i_, v_, o_, ...)                                   \
    {                                                                                             \
        int nvec_ = (vec_ok_) ? (n_) / 4 : 0;                                                     \
        const float4* in4_ = (const float4*)(in_);                                                \
        float4* out4_ = (float4*)(out_);                                                          \
        for (int base_ = tid; base_ < nvec_; base_ += 4 * SB) {                                   \
            float4 ld_[4];                                                                        \
            _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) ld_[u_] = in4_[min(base_ + u_ * SB, nvec_ - 1)]; \
            _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) {                                    \
                if (base_ + u_ * SB < nvec_) {                                                    \
                    float e_[4] = {ld_[u_].x, ld_[u_].y, ld_[u_].z, ld_[u_].w};                   \
                    _Pragma("unroll") for (int c_ = 0; c_ < 4; ++c_) {                            \
                        int i_ = (base_ + u_ * SB) * 4 + c_;                                      \
                        float v_ = e_[c_];                                                        \
                        float o_;                                                                 \
                        __VA_ARGS__                                                               \
                        e_[c_] = o_;                                                              \
                    }                                                                             \
                    out4_[base_ + u_ * SB] = make_float4(e_[0], e_[1], e_[2], e_[3]);             \
                }                                                                                 \
            }                                                                                     \
        }                                                                                         \
        for (int base_ = nvec_ * 4 + tid; base_ < (n_); base_ += 8 * SB) {                        \
            float ld_[8];                                                                         \
            _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_) ld_[u_] = (in_)[min(base_ + u_ * SB, (n_) - 1)]; \
            _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_) {                                    \
                int i_ = base_ + u_ * SB;                                                         \
                if (i_ < (n_)) {                                                                  \
                    float v_ = ld_[u_];                                                           \
                    float o_;                                                                     \
                    __VA_ARGS__                                                                   \
                    (out_)[i_] = o_;                                                              \
                }                                                                                 \
            }                                                                                     \
        }                                                                                         \
    }

// logits [B, V] 32-bit.  Per sequence: temperature, top_k (<= 0: off), top_p (<= 0 or >= 1
// handled as given: off when < 0), u in [0,1), penalty (<= 0: off) with history rows
// hist[b, 0..hist_len[b]).  work [B, V] 32-bit scratch.  out [B] token ids.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, float* __restrict__ work, int vocab,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uniform,
              const float* __restrict__ penalty, const int* __restrict__ hist, int hist_stride,
              const int* __restrict__ hist_len, int* __restrict__ out) {
    constexpr int SB = SAMPLE_THREADS;
    __shared__ ArgMax am_scratch[SB / 64];
    __shared__ float f_scratch[SB / 64];
    constexpr int WAVES = SB / 64;
    constexpr int TIE_CAP = 1024, PEN_WORDS = 2048, PEN_HIST = 256, MAX_CHUNKS = SAMPLE_MAX_VOCAB / 256;
    __shared__ int tie_idx[TIE_CAP];
    __shared__ int n_ties;
    __shared__ unsigned pen_bits[PEN_WORDS];
    __shared__ int pen_hist[PEN_HIST];                 // the history, when it fits: a token that pays for the walk pays LDS reads, not trips to memory
    __shared__ float chunk_sum[MAX_CHUNKS];
    __shared__ float seg_base;
    __shared__ __align__(8) unsigned hist_cnt[WAVES * 256 * 2];   // a histogram per wave: counts, or 64-bit masses
    __shared__ __align__(8) unsigned bin_cnt[256 * 2];
    __shared__ int pick[2];
    __shared__ unsigned long long pick64[2];
    int b = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)b * vocab;
    float* wrow = work + (size_t)b * vocab;
    float pen = penalty ? penalty[b] : 0.f;
    bool use_pen = pen > 0.f && fabsf(pen - 1.0f) >= 1.1920929e-07f;
    const int* h = hist ? hist + (size_t)b * hist_stride : nullptr;
    int nh = (use_pen && hist_len) ? hist_len[b] : 0;
    float temp = temperature[b];
    float inv_temp = temp > 0.f ? 1.0f / temp : 1.0f;

    // pass 1: penalised, scaled logits into work; maximum and its first index.  A token of the
    // recent history is found through a bitmap over (token mod its size); the few tokens that
    // the bitmap flags are set aside (in the list that later holds the ties) and walk through the
    // history after the pass, a thread each: a walk inside the pass would stand between its
    // batched loads and their use.
    if (nh) {
        for (int i = tid; i < PEN_WORDS; i += SB) pen_bits[i] = 0u;
        if (tid == 0) n_ties = 0;
        __syncthreads();
        for (int j = tid; j < nh; j += SB) {
            int tok = h[j];
            if (j < PEN_HIST) pen_hist[j] = tok;
            unsigned t = (unsigned)tok % (PEN_WORDS * 32);
            atomicOr(&pen_bits[t >> 5], 1u << (t & 31));
        }
        __syncthreads();
        if (nh <= PEN_HIST) h = pen_hist;
    }
    ArgMax best = {-INFINITY, 0x7fffffff};
    bool row_vec = (uintptr_t)row % 16 == 0, work_vec = (uintptr_t)wrow % 16 == 0;
    SAMPLE_ROW_MAP(row, wrow, vocab, row_vec && work_vec, i, v, o,
        bool later = false;
        if (nh) {
            unsigned t = (unsigned)i % (PEN_WORDS * 32);
            if (pen_bits[t >> 5] >> (t & 31) & 1u) {
                int slot = atomicAdd(&n_ties, 1);
                if (slot < TIE_CAP) { tie_idx[slot] = i; later = true; }
                else v = penalised(v, i, h, nh, pen);                           // the list is full: walk here
            }
        }
        if (!later && (v > best.v || best.i == 0x7fffffff)) { best.v = v; best.i = i; }   // a thread meets its indices in growing order
        o = v * inv_temp;
    )
    if (nh) {
        __syncthreads();
        int n_later = min(n_ties, TIE_CAP);
        for (int r = tid; r < n_later; r += SB) {
            int i = tie_idx[r];
            ArgMax mine = {penalised(row[i], i, h, nh, pen), i};
            wrow[i] = mine.v * inv_temp;
            best = better(best, mine);
        }
    }
    best = block_argmax<SB>(best, am_scratch);
    if (!(temp > 0.f)) {
        if (tid == 0) out[b] = best.i == 0x7fffffff ? 0 : best.i;
        return;
    }
    float max_logit = best.v * inv_temp;
    __syncthreads();

    // top-k: the k-th largest value by its ordered key; candidates are the values above it
    // plus, among equal ones, the lowest indices up to k.
    int k = top_k ? top_k[b] : 0;
    uint32_t kth_key = 0;      // everything is a candidate
    int n_above = 0;
    bool limit_k = k > 0 && k < vocab;
    if (limit_k) {
        // the k-th largest key, 8 bits at a time: a histogram of the next 8 bits over the values
        // that match the bits found so far, then the bin that holds the k-th from the top
        uint32_t found = 0;          // leading bits of the k-th key
        int want = k;                // its rank from the top among the values matching them
        for (int level = 0; level < 4; ++level) {
            int shift = 24 - 8 * level;
            for (int i = tid; i < WAVES * 256; i += SB) hist_cnt[i] = 0;
            __syncthreads();
            unsigned* mine = hist_cnt + (tid / 64) * 256;
            SAMPLE_ROW_PASS(wrow, vocab, work_vec, i, v,
                (void)i;
                uint32_t key = float_key(v);
                if (level == 0 || (key >> (shift + 8)) == found) atomicAdd(mine + ((key >> shift) & 255), 1u);
            )
            __syncthreads();
            if (tid < 256) {
                unsigned c = 0;
                for (int w = 0; w < WAVES; ++w) c += hist_cnt[w * 256 + tid];
                bin_cnt[tid] = c;
            }
            __syncthreads();
            if (tid < 64) bin_from_top<unsigned>(bin_cnt, (unsigned)want, tid, &pick[0], (unsigned*)&pick[1]);
            __syncthreads();
            found = (found << 8) | (uint32_t)pick[0];
            want -= pick[1];
            n_above += pick[1];
            __syncthreads();
        }
        kth_key = found;
    }
    // pass 2: probabilities exp(v - max) of candidates into work, zero elsewhere.  Values equal
    // to the k-th one are admitted in index order until k candidates are reached: their indices
    // are collected (there is rarely more than one), ranked among themselves, and the lowest
    // are written back.
    if (tid == 0) n_ties = 0;
    __syncthreads();
    SAMPLE_ROW_MAP(wrow, wrow, vocab, work_vec, i, v, p,
        p = fast_exp(v - max_logit);
        if (limit_k) {
            uint32_t key = float_key(v);
            if (key == kth_key) {
                int slot = atomicAdd(&n_ties, 1);
                if (slot < TIE_CAP) tie_idx[slot] = i;
            }
            if (key <= kth_key) p = 0.f;
        }
    )
    __syncthreads();
    if (limit_k) {
        int ties_allowed = k - n_above, ties = n_ties;
        uint32_t u = (kth_key & 0x80000000u) ? (kth_key & 0x7fffffffu) : ~kth_key;     // the value behind the key
        float p_tie = fast_exp(__uint_as_float(u) - max_logit);
        if (ties <= TIE_CAP) {
            for (int t = tid; t < ties; t += SB) {
                int mine = tie_idx[t], rank = 0;
                for (int j = 0; j < ties; ++j) rank += tie_idx[j] < mine;
                if (rank < ties_allowed) wrow[mine] = p_tie;
            }
        } else if (tid == 0) {
            // a row of thousands of equal values: walk it once, in order
            int admitted = 0;
            for (int i = 0; i < vocab && admitted < ties_allowed; ++i) {
                // the ties are the zeros whose logit has the k-th key; the logits are gone from
                // the work row, but the input row still has them
                float v = row[i];
                if (nh) v = penalised(v, i, h, nh, pen);
                if (float_key(v * inv_temp) == kth_key) { wrow[i] = p_tie; ++admitted; }
            }
        }
        __syncthreads();
    }
    float part = 0.f;
    SAMPLE_ROW_PASS(wrow, vocab, work_vec, i, v, part += v; (void)i;)
    float total = block_sum_f<SB>(part, f_scratch);

    // top-p: smallest set of the most probable candidates with mass >= p * total.
    float p_keep = top_p ? top_p[b] : -1.f;
    if (p_keep >= 0.f && p_keep < 1.0f) {
        // The largest threshold T whose mass(prob >= T) still reaches top_p * total, again 8 bits
        // of the key at a time.  Masses are added as 40-bit fixed-point integers: the order of
        // the additions then does not matter and the same row gives the same choice every time.
        unsigned long long* hist_mass = (unsigned long long*)hist_cnt;      // [WAVES][256] too, twice the bytes
        unsigned long long* bin_mass = (unsigned long long*)bin_cnt;
        unsigned long long my_mass = 0ull;
        SAMPLE_ROW_PASS(wrow, vocab, work_vec, i, p,
            if (p > 0.f) my_mass += (unsigned long long)(p * 1099511627776.0f);   // p * 2^40, p <= 1
            (void)i;
        )
        for (int off = 32; off > 0; off >>= 1) my_mass += __shfl_xor(my_mass, off, 64);
        __syncthreads();
        if ((tid & 63) == 0) bin_mass[tid / 64] = my_mass;
        __syncthreads();
        if (tid == 0) {
            unsigned long long all = 0ull;
            for (int w = 0; w < WAVES; ++w) all += bin_mass[w];
            double t = (double)fminf(fmaxf(p_keep, 0.f), 1.f) * (double)all;
            pick64[0] = t < 1.0 ? 1ull : (unsigned long long)t;     // at least the most probable token
        }
        __syncthreads();
        uint32_t found = 0;
        for (int level = 0; level < 4; ++level) {
            int shift = 24 - 8 * level;
            for (int i = tid; i < WAVES * 256; i += SB) hist_mass[i] = 0ull;
            __syncthreads();
            unsigned long long* mine = hist_mass + (tid / 64) * 256;
            SAMPLE_ROW_PASS(wrow, vocab, work_vec, i, p,
                uint32_t key = float_key(p);
                if (p > 0.f && (level == 0 || (key >> (shift + 8)) == found))
                    atomicAdd(mine + ((key >> shift) & 255u), (unsigned long long)(p * 1099511627776.0f));
                (void)i;
            )
            __syncthreads();
            if (tid < 256) {
                unsigned long long c = 0;
                for (int w = 0; w < WAVES; ++w) c += hist_mass[w * 256 + tid];
                bin_mass[tid] = c;
            }
            __syncthreads();
            if (tid < 64) bin_from_top<unsigned long long>(bin_mass, pick64[0], tid, &pick[0], &pick64[1]);
            __syncthreads();
            if (tid == 0) pick64[0] -= pick64[1];
            found = (found << 8) | (uint32_t)pick[0];
            __syncthreads();
        }
        uint32_t lo = found;
        float kept = 0.f;
        SAMPLE_ROW_MAP(wrow, wrow, vocab, work_vec, i, p, q,
            q = (p > 0.f && float_key(p) >= lo) ? p : 0.f;
            kept += q;
            (void)i;
        )
        __syncthreads();
        total = block_sum_f<SB>(kept, f_scratch);
    }

    // draw: the first index at which the cumulative mass, in index order, reaches u * total.
    // The row is cut into chunks of 256 values (4 consecutive ones per lane); every wave adds up
    // its chunks, one thread walks the chunk sums to the chunk that holds the index, and the
    // first wave finds the index inside it with a scan over the lanes.
    float threshold = uniform[b] * fmaxf(total, 1.17549435e-38f);
    int n_chunks = (vocab + 255) / 256;
    int lane = tid & 63, wave = tid / 64;
    for (int c = wave; c < n_chunks; c += WAVES) {
        int i0 = c * 256 + lane * 4;
        float sum = 0.f;
        if (work_vec && i0 + 3 < vocab) {
            float4 q = *(const float4*)(wrow + i0);
            sum = ((q.x + q.y) + q.z) + q.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) sum += i0 + e < vocab ? wrow[i0 + e] : 0.f;
        }
        sum = wave_sum(sum);
        if (lane == 0) chunk_sum[c] = sum;
    }
    __syncthreads();
    if (wave == 0) {
        // the chunk in which the cumulative mass reaches the threshold: every lane adds up a run
        // of consecutive chunk sums, a scan over the lanes finds the run, its lane walks it
        int run = (n_chunks + 63) / 64, c0 = lane * run, c1 = min(n_chunks, c0 + run);
        float mine = 0.f;
        for (int c = c0; c < c1; ++c) mine += chunk_sum[c];
        float upto = mine;                                   // inclusive scan over the lanes
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            float o = __shfl_up(upto, off, 64);
            if (lane >= off) upto += o;
        }
        unsigned long long reach = __builtin_amdgcn_ballot_w64(mine > 0.f && upto >= threshold);
        int owner = reach ? __builtin_ctzll(reach) : -1;     // the first lane whose run reaches it
        if (owner < 0 && lane == 0) pick[0] = n_chunks;
        if (lane == owner) {
            float acc = upto - mine;
            int c = c0;
            for (; c < c1; ++c) {
                if (chunk_sum[c] > 0.f && acc + chunk_sum[c] >= threshold) break;
                acc += chunk_sum[c];
            }
            if (c == c1) {                                   // rounding inside the run: its last chunk with mass
                for (c = c1 - 1; c > c0 && !(chunk_sum[c] > 0.f); --c) {}
                acc = upto - mine;
                for (int j = c0; j < c; ++j) acc += chunk_sum[j];
            }
            pick[0] = c;
            seg_base = acc;
        }
    }
    __syncthreads();
    if (wave == 0) {
        int c = pick[0], chosen = 0x7fffffff, last_positive = -1;
        if (c < n_chunks) {
            int i0 = c * 256 + lane * 4;
            float v[4], mine = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = i0 + e < vocab ? wrow[i0 + e] : 0.f; mine += v[e]; }
            float before = mine;                                // inclusive scan over the lanes
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                float o = __shfl_up(before, off, 64);
                if (lane >= off) before += o;
            }
            float acc = seg_base + (before - mine);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (v[e] > 0.f) {
                    acc += v[e];
                    last_positive = i0 + e;
                    if (acc >= threshold && chosen == 0x7fffffff) chosen = i0 + e;
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            chosen = min(chosen, __shfl_xor(chosen, off, 64));
            last_positive = max(last_positive, __shfl_xor(last_positive, off, 64));
        }
        // the chunk's sum was added up in another order than the scan: if rounding leaves the scan
        // short of the threshold, the chunk's last candidate is meant; without any chunk (the
        // threshold above the total by rounding) the most probable token
        if (lane == 0) out[b] = chosen != 0x7fffffff ? chosen : (last_positive >= 0 ? last_positive : best.i);
    }
}

// ---- a small top-k: slices, then one wave ------------------------------------------------------
// With a top-k of at most SMALL_K everything after the selection concerns k candidates, and the
// selection splits: the vocabulary is cut into at most 64 slices, a block per slice and sequence
// keeps its slice in registers (penalty and temperature applied) and hands out its k best in
// order (value descending, then index ascending: the order in which ties are admitted); the k
// best of the row are among these.  One wave per sequence then merges the sorted lists, a lane
// per slice, and lane r ends up with the r-th best: softmax, top-p and the draw are a matter of
// shuffles.  The rules are those of sample_kernel above; a row is read once, by many CUs,
// instead of a dozen times by one.
constexpr int SMALL_K = 64, SLICE_THREADS = 256, MAX_SLICES = 64;

template <int EPT>
__global__ void __launch_bounds__(SLICE_THREADS)
sample_slice_topk_kernel(const float* __restrict__ logits, int vocab, int slice_len,
                         const float* __restrict__ temperature, const int* __restrict__ top_k,
                         const float* __restrict__ penalty, const int* __restrict__ hist, int hist_stride,
                         const int* __restrict__ hist_len, int k_stride, float* __restrict__ cand_v,
                         int* __restrict__ cand_i) {
    __shared__ ArgMax am_scratch[SLICE_THREADS / 64];
    int s = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    int base = s * slice_len, end = min(vocab, base + slice_len);
    float temp = temperature[b];
    bool greedy = !(temp > 0.f);
    float inv_temp = greedy ? 1.0f : 1.0f / temp;
    int k = greedy ? 1 : min(max(top_k[b], 1), k_stride);
    const float* row = logits + (size_t)b * vocab;
    float v[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        int i = base + e * SLICE_THREADS + tid;
        v[e] = i < end ? row[i] : -INFINITY;
    }
    float pen = penalty ? penalty[b] : 0.f;
    if (pen > 0.f && fabsf(pen - 1.0f) >= 1.1920929e-07f && hist && hist_len) {
        // once per occurrence in the history, as the reference does; the thread that holds the
        // token applies it
        const int* h = hist + (size_t)b * hist_stride;
        int nh = hist_len[b];
        for (int j = 0; j < nh; ++j) {
            int off = h[j] - base;
            if (off >= 0 && off < end - base && off % SLICE_THREADS == tid) {
                int we = off / SLICE_THREADS;
#pragma unroll
                for (int e = 0; e < EPT; ++e)
                    if (e == we) v[e] = v[e] > 0.f ? v[e] / pen : v[e] * pen;
            }
        }
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[e] *= inv_temp;     // (-inf stays -inf)
    float* out_v = cand_v + ((size_t)b * gridDim.x + s) * k_stride;
    int* out_i = cand_i + ((size_t)b * gridDim.x + s) * k_stride;
    for (int r = 0; r < k; ++r) {
        // a thread's indices grow with e: its first maximum is its lowest index
        ArgMax mine = {-INFINITY, 0x7fffffff};
#pragma unroll
        for (int e = 0; e < EPT; ++e)
            if (v[e] > mine.v) { mine.v = v[e]; mine.i = base + e * SLICE_THREADS + tid; }
        ArgMax win = block_argmax<SLICE_THREADS>(mine, am_scratch);
        if (tid == 0) { out_v[r] = win.v; out_i[r] = win.i; }
        if (win.i == 0x7fffffff) {                      // the slice is used up: the rest of the list is empty
            for (int q = r + 1 + tid; q < k; q += SLICE_THREADS) { out_v[q] = -INFINITY; out_i[q] = 0x7fffffff; }
            break;
        }
        if ((win.i - base) % SLICE_THREADS == tid) {
            int we = (win.i - base) / SLICE_THREADS;
#pragma unroll
            for (int e = 0; e < EPT; ++e)
                if (e == we) v[e] = -INFINITY;
        }
    }
}

__global__ void __launch_bounds__(64)
sample_merge_draw_kernel(const float* __restrict__ cand_v, const int* __restrict__ cand_i, int n_slices,
                         int k_stride, const float* __restrict__ temperature, const int* __restrict__ top_k,
                         const float* __restrict__ top_p, const float* __restrict__ uniform,
                         int* __restrict__ out) {
    __shared__ float sv[MAX_SLICES * SMALL_K];
    __shared__ int si[MAX_SLICES * SMALL_K];
    int b = blockIdx.x, lane = threadIdx.x;
    float temp = temperature[b];
    bool greedy = !(temp > 0.f);
    int k = greedy ? 1 : min(max(top_k[b], 1), k_stride);
    for (int idx = lane; idx < n_slices * k; idx += 64) {
        int s = idx / k, r = idx - s * k;
        sv[s * SMALL_K + r] = cand_v[((size_t)b * n_slices + s) * k_stride + r];
        si[s * SMALL_K + r] = cand_i[((size_t)b * n_slices + s) * k_stride + r];
    }
    __syncthreads();
    // merge of the sorted lists, a lane per slice: lane r keeps the r-th best of the row
    int ptr = 0;
    ArgMax mine = {-INFINITY, 0x7fffffff};
    for (int r = 0; r < k; ++r) {
        ArgMax head = {-INFINITY, 0x7fffffff};
        if (lane < n_slices && ptr < k) { head.v = sv[lane * SMALL_K + ptr]; head.i = si[lane * SMALL_K + ptr]; }
        ArgMax win = head;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            ArgMax o;
            o.v = __shfl_xor(win.v, off, 64);
            o.i = __shfl_xor(win.i, off, 64);
            win = better(win, o);
        }
        if (win.i != 0x7fffffff && head.i == win.i) ++ptr;
        if (lane == r) mine = win;
    }
    if (greedy) {
        if (lane == 0) out[b] = mine.i == 0x7fffffff ? 0 : mine.i;
        return;
    }
    bool valid = lane < k && mine.i != 0x7fffffff;
    float top_v = __shfl(mine.v, 0, 64);
    float p = valid ? fast_exp(mine.v - top_v) : 0.f;
    // top-p over the candidates in descending order: the shortest prefix whose mass reaches
    // top_p of the total, and every candidate as probable as its last one
    bool keep = valid;
    float tp = top_p ? top_p[b] : -1.0f;
    if (tp >= 0.f && tp < 1.0f) {
        double cum = (double)p;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            double o = __shfl_up(cum, off, 64);
            if (lane >= off) cum += o;
        }
        double total = __shfl(cum, 63, 64);
        unsigned long long reached = __builtin_amdgcn_ballot_w64(valid && cum >= (double)tp * total);
        unsigned long long any = __builtin_amdgcn_ballot_w64(valid);
        int cut = reached ? __builtin_ctzll(reached) : (any ? 63 - __builtin_clzll(any) : 0);
        float last_p = __shfl(p, cut, 64);
        keep = valid && p >= last_p;
    }
    // the draw walks the kept candidates in index order
    double below = 0.0, total_kept = 0.0;
    for (int j = 0; j < k; ++j) {
        float pj = __shfl(p, j, 64);
        int ij = __shfl(mine.i, j, 64);
        bool kj = __shfl((int)keep, j, 64) != 0;
        if (kj) {
            total_kept += (double)pj;
            if (ij < mine.i) below += (double)pj;
        }
    }
    double t = (double)uniform[b] * total_kept;
    unsigned long long hit = __builtin_amdgcn_ballot_w64(keep && below <= t && t < below + (double)p);
    // (a threshold at or above the total by rounding means the last kept candidate in index order)
    int chosen;
    if (hit) {
        chosen = __shfl(mine.i, __builtin_ctzll(hit), 64);
    } else {
        int cand = keep ? mine.i : -1;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cand = max(cand, __shfl_xor(cand, off, 64));
        chosen = cand >= 0 ? cand : (__shfl(mine.i, 0, 64) == 0x7fffffff ? 0 : __shfl(mine.i, 0, 64));
    }
    if (lane == 0) out[b] = chosen;
}

// small_k: 0, or a bound (at most SMALL_K) that every sequence's top_k lies in [1, small_k] under
// (sequences with a temperature <= 0 aside): then the slice kernels run, if the workspace holds
// their candidate lists.
ROCML_EXPORT int rocml_sample(const float* logits, float* work, int batch, int vocab,
                              const float* temperature, const int* top_k, const float* top_p,
                              const float* uniform, const float* penalty, const int* hist,
                              int hist_stride, const int* hist_len, int small_k, int* out, hipStream_t stream) {
    ROCML_REQUIRE(batch >= 0 && vocab > 0, "sample: bad sizes B=%d V=%d", batch, vocab);
    ROCML_REQUIRE(logits && work && temperature && uniform && out, "sample: null argument");
    ROCML_REQUIRE(vocab <= SAMPLE_MAX_VOCAB, "sample: vocabulary %d exceeds %d", vocab, SAMPLE_MAX_VOCAB);
    ROCML_REQUIRE(small_k >= 0 && small_k <= SMALL_K && (small_k == 0 || top_k), "sample: bad top-k bound %d", small_k);
    if (batch == 0) return 0;
    if (small_k > 0) {
        // slices of 4096 values (16 per thread), or of 16384 for the largest vocabularies
        int ept = vocab <= MAX_SLICES * SLICE_THREADS * 16 ? 16 : 64;
        int slice_len = SLICE_THREADS * ept;
        int n_slices = (vocab + slice_len - 1) / slice_len;
        if (n_slices <= MAX_SLICES && (long long)n_slices * small_k * 8 <= (long long)vocab * 4) {
            float* cand_v = work;
            int* cand_i = (int*)(work + (size_t)batch * n_slices * small_k);
            dim3 grid(n_slices, batch);
            if (ept == 16)
                sample_slice_topk_kernel<16><<<grid, SLICE_THREADS, 0, stream>>>(
                    logits, vocab, slice_len, temperature, top_k, penalty, hist, hist_stride, hist_len, small_k, cand_v, cand_i);
            else
                sample_slice_topk_kernel<64><<<grid, SLICE_THREADS, 0, stream>>>(
                    logits, vocab, slice_len, temperature, top_k, penalty, hist, hist_stride, hist_len, small_k, cand_v, cand_i);
            sample_merge_draw_kernel<<<batch, 64, 0, stream>>>(cand_v, cand_i, n_slices, small_k, temperature, top_k,
                                                               top_p, uniform, out);
            ROCML_CHECK_LAUNCH("sample");
            return 0;
        }
    }
    sample_kernel<<<batch, SAMPLE_THREADS, 0, stream>>>(logits, work, vocab, temperature, top_k, top_p, uniform,
                                            penalty, hist, hist_stride, hist_len, out);
    ROCML_CHECK_LAUNCH("sample");
    return 0;
}

// Greedy only: out[b] = first index of the maximum of logits[b, :].
__global__ void __launch_bounds__(SB)
argmax_kernel(const float* __restrict__ logits, int vocab, int* __restrict__ out) {
    __shared__ ArgMax am_scratch[SB / 64];
    int b = blockIdx.x;
    const float* row = logits + (size_t)b * vocab;
    ArgMax best = {-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < vocab; i += SB) {
        ArgMax c = {row[i], i};
        best = better(best, c);
    }
    best = block_argmax(best, am_scratch);
    if (threadIdx.x == 0) out[b] = best.i == 0x7fffffff ? 0 : best.i;
}

// Two stages for long rows: a row is cut into ARGMAX_CHUNKS pieces, each block finds its piece's
// first maximum, a second kernel picks among the pieces (lower piece wins a tie, so the first
// maximum of the row wins).  One block per row would read a 150k-entry row alone.
constexpr int ARGMAX_CHUNKS = 32;

__global__ void __launch_bounds__(SB)
argmax_partial_kernel(const float* __restrict__ logits, int vocab, float* __restrict__ part_val,
                      int* __restrict__ part_idx) {
    __shared__ ArgMax am_scratch[SB / 64];
    int b = blockIdx.y, c = blockIdx.x;
    int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    int lo = c * per, hi = min(vocab, lo + per);
    const float* row = logits + (size_t)b * vocab;
    ArgMax best = {-INFINITY, 0x7fffffff};
    for (int i = lo + threadIdx.x; i < hi; i += SB) {
        ArgMax cand = {row[i], i};
        best = better(best, cand);
    }
    best = block_argmax(best, am_scratch);
    if (threadIdx.x == 0) {
        part_val[b * ARGMAX_CHUNKS + c] = best.v;
        part_idx[b * ARGMAX_CHUNKS + c] = best.i;
    }
}

__global__ void argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                                    int* __restrict__ out) {
    int b = blockIdx.x, lane = threadIdx.x;      // 64 threads
    ArgMax a = {-INFINITY, 0x7fffffff};
    if (lane < ARGMAX_CHUNKS) a = ArgMax{part_val[b * ARGMAX_CHUNKS + lane], part_idx[b * ARGMAX_CHUNKS + lane]};
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        ArgMax o;
        o.v = __shfl_xor(a.v, off, 64);
        o.i = __shfl_xor(a.i, off, 64);
        a = better(a, o);
    }
    if (lane == 0) out[b] = a.i == 0x7fffffff ? 0 : a.i;
}

// work: 2 * batch * ARGMAX_CHUNKS 32-bit words of device memory, or null for the one-stage kernel.
ROCML_EXPORT int rocml_argmax(const float* logits, int batch, int vocab, int* out, void* work,
                              hipStream_t stream) {
    ROCML_REQUIRE(batch >= 0 && vocab > 0, "argmax: bad sizes B=%d V=%d", batch, vocab);
    if (batch == 0) return 0;
    if (work && vocab >= 4096) {
        float* part_val = (float*)work;
        int* part_idx = (int*)work + (size_t)batch * ARGMAX_CHUNKS;
        argmax_partial_kernel<<<dim3(ARGMAX_CHUNKS, batch), SB, 0, stream>>>(logits, vocab, part_val, part_idx);
        argmax_final_kernel<<<batch, 64, 0, stream>>>(part_val, part_idx, out);
    } else {
        argmax_kernel<<<batch, SB, 0, stream>>>(logits, vocab, out);
    }
    ROCML_CHECK_LAUNCH("argmax");
    return 0;
}

// ---- the same without a workspace and without allocating ------------------------------------
// The partial maxima of rocml_argmax's first stage, in memory of the library itself.  In host
// code the array's name is not a device address; the address on each GPU is asked for once, with
// that GPU current, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) uint32_t g_argmax_static_scratch[2 * ROCML_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS];

constexpr int STATIC_MAX_DEVICES = 64;
static void* g_argmax_static_ptr[STATIC_MAX_DEVICES] = {};
static std::mutex g_argmax_static_lock;

static int argmax_static_scratch(void** ptr) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return rocml_fail("argmax_static: no current device: %s", hipGetErrorString(e));
    if (device < 0 || device >= STATIC_MAX_DEVICES)
        return rocml_fail("argmax_static: device %d is beyond the %d this library keeps an address for", device, STATIC_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_argmax_static_lock);
    if (!g_argmax_static_ptr[device]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_argmax_static_scratch));
        if (e != hipSuccess || !p)
            return rocml_fail("argmax_static: cannot find the scratch array on device %d: %s", device, hipGetErrorString(e));
        g_argmax_static_ptr[device] = p;
    }
    *ptr = g_argmax_static_ptr[device];
    return 0;
}

ROCML_EXPORT int rocml_argmax_static(const float* logits, int batch, int vocab, int* out, hipStream_t stream) {
    ROCML_REQUIRE(batch >= 0 && vocab > 0, "argmax_static: bad sizes B=%d V=%d", batch, vocab);
    ROCML_REQUIRE(batch <= ROCML_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows exceed the %d the library's scratch array holds",
                  batch, ROCML_ARGMAX_STATIC_MAX_ROWS);
    ROCML_REQUIRE(logits && out, "argmax_static: null pointer");
    if (batch == 0) return 0;
    void* work = nullptr;
    if (argmax_static_scratch(&work)) return 1;
    float* part_val = (float*)work;
    int* part_idx = (int*)work + (size_t)batch * ARGMAX_CHUNKS;
    argmax_partial_kernel<<<dim3(ARGMAX_CHUNKS, batch), SB, 0, stream>>>(logits, vocab, part_val, part_idx);
    argmax_final_kernel<<<batch, 64, 0, stream>>>(part_val, part_idx, out);
    ROCML_CHECK_LAUNCH("argmax_static");
    return 0;
}
