// Sampling on the device, one 256-thread block per sequence, in the order of the reference's
// host sampler (rocml/src/sample.rs:90-166): repeat penalty over recent history, greedy if the
// temperature is not positive (first maximum wins, :172-182), else scale by 1/temperature,
// keep the top k, softmax, keep the smallest set of most probable tokens whose mass reaches
// top_p, draw with the caller's uniform number.
#include "common.h"

ROCML_LAST_ERROR_FN(sampling)

constexpr int SB = 256;

struct ArgMax { float v; int i; };

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
    // larger value wins; on a tie the lower index wins ("first maximum").
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

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
    for (int w = 1; w < SB / 64; ++w) r = better(r, scratch[w]);
    return r;
}

__device__ float block_sum_f(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < SB / 64; ++w) r += scratch[w];
    return r;
}

__device__ int block_sum_i(int v, int* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x / 64] = v;
    __syncthreads();
    int r = 0;
#pragma unroll
    for (int w = 0; w < SB / 64; ++w) r += scratch[w];
    return r;
}

// Order-preserving map of a float to an unsigned key (larger float -> larger key).
__device__ __forceinline__ uint32_t float_key(float f) {
    uint32_t u = __float_as_uint(f);
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

// logits [B, V] 32-bit.  Per sequence: temperature, top_k (<= 0: off), top_p (<= 0 or >= 1
// handled as given: off when < 0), u in [0,1), penalty (<= 0: off) with history rows
// hist[b, 0..hist_len[b]).  work [B, V] 32-bit scratch.  out [B] token ids.
__global__ void __launch_bounds__(SB)
sample_kernel(const float* __restrict__ logits, float* __restrict__ work, int vocab,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uniform,
              const float* __restrict__ penalty, const int* __restrict__ hist, int hist_stride,
              const int* __restrict__ hist_len, int* __restrict__ out) {
    __shared__ ArgMax am_scratch[SB / 64];
    __shared__ float f_scratch[SB / 64];
    __shared__ int i_scratch[SB / 64];
    __shared__ float seg_sum[SB];
    __shared__ int seg_cnt[SB];
    int b = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)b * vocab;
    float* wrow = work + (size_t)b * vocab;
    float pen = penalty ? penalty[b] : 0.f;
    bool use_pen = pen > 0.f && fabsf(pen - 1.0f) >= 1.1920929e-07f;
    const int* h = hist ? hist + (size_t)b * hist_stride : nullptr;
    int nh = (use_pen && hist_len) ? hist_len[b] : 0;
    float temp = temperature[b];
    float inv_temp = temp > 0.f ? 1.0f / temp : 1.0f;

    // pass 1: penalised, scaled logits into work; maximum and its first index.
    ArgMax best = {-INFINITY, 0x7fffffff};
    for (int i = tid; i < vocab; i += SB) {
        float v = row[i];
        if (nh) v = penalised(v, i, h, nh, pen);
        ArgMax c = {v, i};
        best = better(best, c);
        wrow[i] = v * inv_temp;
    }
    best = block_argmax(best, am_scratch);
    if (!(temp > 0.f)) {
        if (tid == 0) out[b] = best.i == 0x7fffffff ? 0 : best.i;
        return;
    }
    float max_logit = best.v * inv_temp;
    __syncthreads();

    // top-k: binary search over the ordered keys for the k-th largest value; candidates are
    // the values above it plus, among equal ones, the lowest indices up to k.
    int k = top_k ? top_k[b] : 0;
    uint32_t kth_key = 0;      // everything is a candidate
    int n_above = 0;
    bool limit_k = k > 0 && k < vocab;
    if (limit_k) {
        uint32_t lo = 0, hi = 0xffffffffu;   // find largest key T with count(key >= T) >= k
        while (lo < hi) {
            uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) / 2);
            int cnt = 0;
            for (int i = tid; i < vocab; i += SB) cnt += float_key(wrow[i]) >= mid;
            cnt = block_sum_i(cnt, i_scratch);
            if (cnt >= k) lo = mid; else hi = mid - 1;
        }
        kth_key = lo;
        int cnt = 0;
        for (int i = tid; i < vocab; i += SB) cnt += float_key(wrow[i]) > kth_key;
        n_above = block_sum_i(cnt, i_scratch);
    }
    // pass 2: probabilities exp(v - max) of candidates into work, zero elsewhere.  Values equal
    // to the k-th one are admitted in index order until k candidates are reached: every thread
    // owns a contiguous segment, counts its ties, and admits those whose rank is below the rest.
    int per = (vocab + SB - 1) / SB;
    int s0 = min(vocab, tid * per), s1 = min(vocab, s0 + per);
    if (limit_k) {
        int ties_allowed = k - n_above;
        int mine = 0;
        for (int i = s0; i < s1; ++i) mine += float_key(wrow[i]) == kth_key;
        seg_cnt[tid] = mine;
        __syncthreads();
        int before = 0;
        for (int t = 0; t < tid; ++t) before += seg_cnt[t];
        for (int i = s0; i < s1; ++i) {
            float v = wrow[i];
            uint32_t key = float_key(v);
            bool keep = key > kth_key || (key == kth_key && before++ < ties_allowed);
            wrow[i] = keep ? expf(v - max_logit) : 0.f;
        }
    } else {
        for (int i = s0; i < s1; ++i) wrow[i] = expf(wrow[i] - max_logit);
    }
    __syncthreads();
    float part = 0.f;
    for (int i = tid; i < vocab; i += SB) part += wrow[i];
    float total = block_sum_f(part, f_scratch);

    // top-p: smallest set of the most probable candidates with mass >= p * total.  Binary
    // search for the largest probability threshold whose mass still reaches it.
    float p_keep = top_p ? top_p[b] : -1.f;
    if (p_keep >= 0.f && p_keep < 1.0f) {
        float target = fminf(fmaxf(p_keep, 0.f), 1.f) * total;
        uint32_t lo = 0, hi = float_key(1.0f);
        // largest T with mass(prob >= T) >= target
        while (lo < hi) {
            uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) / 2);
            float mass = 0.f;
            for (int i = tid; i < vocab; i += SB) { float p = wrow[i]; if (p > 0.f && float_key(p) >= mid) mass += p; }
            mass = block_sum_f(mass, f_scratch);
            if (mass >= target) lo = mid; else hi = mid - 1;
        }
        float kept = 0.f;
        for (int i = tid; i < vocab; i += SB) {
            float p = wrow[i];
            if (!(p > 0.f && float_key(p) >= lo)) { p = 0.f; wrow[i] = 0.f; }
            kept += p;
        }
        __syncthreads();
        total = block_sum_f(kept, f_scratch);
    }

    // draw: walk the cumulative mass in index order until it reaches u * total.
    float threshold = uniform[b] * fmaxf(total, 1.17549435e-38f);
    float seg = 0.f;
    for (int i = s0; i < s1; ++i) seg += wrow[i];
    seg_sum[tid] = seg;
    __syncthreads();
    if (tid == 0) {
        float acc = 0.f;
        int chosen = -1;
        for (int t = 0; t < SB && chosen < 0; ++t) {
            if (acc + seg_sum[t] >= threshold && seg_sum[t] > 0.f) {
                int a0 = min(vocab, t * per), a1 = min(vocab, a0 + per);
                for (int i = a0; i < a1; ++i) {
                    float p = wrow[i];
                    if (p > 0.f) { acc += p; if (acc >= threshold) { chosen = i; break; } }
                }
            } else {
                acc += seg_sum[t];
            }
        }
        if (chosen < 0) chosen = best.i;   // rounding left the threshold above the total
        out[b] = chosen;
    }
}

ROCML_EXPORT int rocml_sample(const float* logits, float* work, int batch, int vocab,
                              const float* temperature, const int* top_k, const float* top_p,
                              const float* uniform, const float* penalty, const int* hist,
                              int hist_stride, const int* hist_len, int* out, hipStream_t stream) {
    ROCML_REQUIRE(batch >= 0 && vocab > 0, "sample: bad sizes B=%d V=%d", batch, vocab);
    ROCML_REQUIRE(logits && work && temperature && uniform && out, "sample: null argument");
    if (batch == 0) return 0;
    sample_kernel<<<batch, SB, 0, stream>>>(logits, work, vocab, temperature, top_k, top_p, uniform,
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
