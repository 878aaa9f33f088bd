// bfloat16 matrix products on the gfx950 matrix cores: out[M,N] (+)= X[M,K] * W[N,K]^T with
// 32-bit accumulation.  Both operands are K-contiguous, which is what an MFMA lane wants: 8
// consecutive K values (16 bytes) of one row.
//
// Two kernels:
//  * gemm_mfma_kernel, many rows (prefill): 128x128 output tile per 256-thread block, four
//    waves in 2x2, each wave 64x64 = 2x2 tiles of v_mfma_f32_32x32x16_bf16; K staged 64 at a
//    time through double-buffered LDS with one barrier per stage; rows padded by 16 bytes so
//    that 128-bit LDS reads of 16 rows fall into 16 different bank groups.  The idea of the
//    tiling (big tile per block, 2x2 fragments per wave, padded double-buffered LDS) is the
//    reference's WMMA kernel (rocml-kernels/kernels/gemm_xwt_wmma_impl.h:211-378); layouts and
//    sizes are for wave64 MFMA.  Blocks are renumbered so that each of the 8 XCDs works on a
//    contiguous range of tiles and its L2 sees few weight panels.
//  * gemm_skinny_kernel, few rows (decode, M <= 64): memory-bound; a block owns 64 weight rows
//    and a K range, each wave 16 rows.  Weights go straight from global memory into MFMA
//    operand registers (v_mfma_f32_16x16x32_bf16), 8 loads of 16 bytes in flight per lane; the
//    activations of the K range are shared through LDS.  Split-K partial sums go to a
//    workspace and are added in split order by a second kernel, so results do not depend on
//    timing (rocml-kernels/kernels/gemm_splitk_reduce.hip:4-10 has the same rule).
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // 16 bytes as a native vector: a
// conditional between two of these is a register select, between two uint4 structs it goes
// through memory and drags whole arrays into scratch

__device__ __forceinline__ bf16x8_t as_frag(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ __forceinline__ bf16x8_t as_frag4(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

// Unconditional 16-byte load from an address the caller has clamped into range, zeroed
// afterwards when the element is outside the matrix: a load under a branch would be waited for
// before the next one is issued.
__device__ __forceinline__ uint4 load16_or_zero(const bf16_t* p, bool ok) {
    uint4 v = *(const uint4*)p;
    v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
    return v;
}

// EPI_SWIGLU: weight rows come in pairs (gate_j, up_j); the output is bfloat16 [M, N/2] with
// out[m][j] = silu(gate) * up (rocml-kernels/kernels/silu_mul.hip:12-20), formed from the 32-bit
// accumulators so that gate and up are never rounded or written.
enum GemmEpilogue : int { EPI_F32 = 0, EPI_BF16 = 1, EPI_ACC = 2, EPI_SWIGLU = 3 };

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

template <int EPI>
__device__ __forceinline__ void epilogue_store(void* out, size_t idx, float v) {
    if (EPI == EPI_F32) ((float*)out)[idx] = v;
    else if (EPI == EPI_BF16) ((bf16_t*)out)[idx] = f32_to_bf16(v);
    else if (EPI == EPI_ACC) ((float*)out)[idx] += v;
}

// ---- many rows ---------------------------------------------------------------------------
// One kernel, two shapes (see GemmTile below): 128x128 with four waves for most products, and
// 256x256 with eight waves (two per SIMD, each 128x64) for products wide enough to give every
// CU several such tiles: four times the products per LDS byte and per barrier.
constexpr int GM_BK = 64;
constexpr int GM_ROW = GM_BK / 8 + 1;                 // u32x4_t per LDS row, one of padding

template <int WAVES_M_, int WAVES_N_, int TM_, int TN_>
struct GemmTile {
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;   // waves along M and N
    static constexpr int TM = TM_, TN = TN_;                        // 32x32 MFMA tiles per wave
    static constexpr int BM = WAVES_M * TM * 32, BN = WAVES_N * TN * 32;
    static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    static constexpr int PASS_ROWS = THREADS / 8;                   // tile rows one pass loads
    static constexpr int PA = BM / PASS_ROWS, PB = BN / PASS_ROWS;  // passes per operand
    static constexpr int LDS_BYTES = 2 * (BM + BN) * GM_ROW * 16;   // two stages
};
using GemmTile128 = GemmTile<2, 2, 2, 2>;
using GemmTile256 = GemmTile<2, 4, 4, 2>;

template <int EPI, typename T>
__global__ void __launch_bounds__(T::THREADS)
gemm_mfma_kernel(const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw,
                 void* __restrict__ out, int ldo, int m, int n, int k, int tiles_m, int n_tiles) {
    extern __shared__ u32x4_t gm_smem[];              // [2 stages][A: BM rows | B: BN rows][GM_ROW]
    constexpr int STAGE = (T::BM + T::BN) * GM_ROW;
    int per_xcd = gridDim.x / 8;
    int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (logical >= n_tiles) return;
    int m0 = (logical % tiles_m) * T::BM, n0 = (logical / tiles_m) * T::BN;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    int lrow = tid >> 3, lkc = tid & 7;
    int nk = (k + GM_BK - 1) / GM_BK;
    // The global loads of the next K stage are issued before the current stage is multiplied
    // and written to the other LDS buffer afterwards: one barrier per stage.  (Loading two
    // stages ahead was tried: the compiler then keeps two sets of accumulators and the kernel
    // is slower.)
    u32x4_t ra[T::PA], rb[T::PB];
    f32x16_t acc[T::TM][T::TN];
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // Loads go to clamped addresses and are used as they come: rows beyond M or N only feed
    // outputs that are never stored.  Only a 16-byte piece beyond K must count as zero, and that
    // is decided when the piece is written to LDS, long after the load was issued (a select
    // right behind the load would make the wave wait for it there).
    const bf16_t* xrow[T::PA];
    const bf16_t* wrow[T::PB];
#pragma unroll
    for (int i = 0; i < T::PA; ++i) xrow[i] = x + (size_t)min(m0 + lrow + T::PASS_ROWS * i, m - 1) * ldx;
#pragma unroll
    for (int i = 0; i < T::PB; ++i) wrow[i] = w + (size_t)min(n0 + lrow + T::PASS_ROWS * i, n - 1) * ldw;
    // Written as macros over the register arrays: handed to a function through a pointer, the
    // arrays would be kept in scratch memory and every load waited for at once.
#define GM_LOAD_GLOBAL(kt_)                                                                      \
    {                                                                                            \
        int gk_ = (kt_) * GM_BK + lkc * 8;                                                       \
        gk_ = gk_ < k ? gk_ : 0;                                                                 \
        _Pragma("unroll") for (int i = 0; i < T::PA; ++i) ra[i] = *(const u32x4_t*)(xrow[i] + gk_); \
        _Pragma("unroll") for (int i = 0; i < T::PB; ++i) rb[i] = *(const u32x4_t*)(wrow[i] + gk_); \
    }
#define GM_STORE_LDS(kt_, buf_)                                                                  \
    {                                                                                            \
        u32x4_t* sa_ = gm_smem + (buf_) * STAGE;                                                 \
        u32x4_t* sb_ = sa_ + T::BM * GM_ROW;                                                     \
        bool kin_ = (kt_) * GM_BK + lkc * 8 < k;                                                 \
        const u32x4_t zero_ = {0u, 0u, 0u, 0u};                                                  \
        _Pragma("unroll") for (int i = 0; i < T::PA; ++i)                                        \
            sa_[(lrow + T::PASS_ROWS * i) * GM_ROW + lkc] = kin_ ? ra[i] : zero_;                \
        _Pragma("unroll") for (int i = 0; i < T::PB; ++i)                                        \
            sb_[(lrow + T::PASS_ROWS * i) * GM_ROW + lkc] = kin_ ? rb[i] : zero_;                \
    }
    auto multiply = [&](int buf) {
        const u32x4_t* sa = gm_smem + buf * STAGE;
        const u32x4_t* sb = sa + T::BM * GM_ROW;
#pragma unroll
        for (int kk = 0; kk < GM_BK / 16; ++kk) {
            bf16x8_t a[T::TM], b[T::TN];
            int col = kk * 2 + (lane >> 5);
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
                a[i] = as_frag4(sa[(wm * T::TM * 32 + i * 32 + (lane & 31)) * GM_ROW + col]);
#pragma unroll
            for (int j = 0; j < T::TN; ++j)
                b[j] = as_frag4(sb[(wn * T::TN * 32 + j * 32 + (lane & 31)) * GM_ROW + col]);
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
#pragma unroll
                for (int j = 0; j < T::TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    };

    GM_LOAD_GLOBAL(0)
    GM_STORE_LDS(0, 0)
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        int buf = kt & 1;
        bool more = kt + 1 < nk;
        if (more) GM_LOAD_GLOBAL(kt + 1)
        multiply(buf);
        if (more) GM_STORE_LDS(kt + 1, buf ^ 1)
        __syncthreads();
    }
#undef GM_LOAD_GLOBAL
#undef GM_STORE_LDS
    // Accumulator element e of a lane: row 8*(e/4) + 4*(lane/32) + e%4, column lane%32.
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
            int gn = n0 + (wn * T::TN + j) * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int gm = m0 + (wm * T::TM + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (EPI == EPI_SWIGLU) {
                    // neighbouring lanes hold neighbouring columns: the even one has the gate
                    float other = __shfl_xor(acc[i][j][e], 1, 64);
                    if ((lane & 1) == 0 && gm < m && gn + 1 < n)
                        ((bf16_t*)out)[(size_t)gm * ldo + (gn >> 1)] = f32_to_bf16(silu_mul(acc[i][j][e], other));
                } else if (gm < m && gn < n) {
                    epilogue_store<EPI>(out, (size_t)gm * ldo + gn, acc[i][j][e]);
                }
            }
        }
}

// ---- few rows ----------------------------------------------------------------------------
constexpr int GS_BN = 64, GS_KC = 256, GS_THREADS = 256;
constexpr int GS_ROW = GS_KC / 8 + 1;                 // uint4 per LDS row of activations

// PARTIAL: write 32-bit partial sums [split][M][N] instead of the epilogue.
// Loads are never followed by a select: addresses beyond the matrix are clamped to a place
// inside it, rows beyond M or N only feed outputs that are not stored, and a piece beyond K is
// zeroed on the activation side when it is written to LDS (the weight beside it is then some
// finite weight times zero).  A select right behind a load would make the wave wait for the
// load there and undo the overlap of the next chunk's loads with this chunk's products.
template <int MT, int EPI, bool PARTIAL, int WAVES = 4>
__global__ void __launch_bounds__(64 * WAVES)
gemm_skinny_kernel(const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw,
                   void* __restrict__ out, int ldo, int m, int n, int k, int k_per_split) {
    extern __shared__ u32x4_t gs_smem[];              // [2][MT*16][GS_ROW]
    constexpr int ROWS = MT * 16;
    constexpr int THREADS = 64 * WAVES;
    constexpr int XCHUNKS = ROWS * (GS_KC / 8) / THREADS;   // 16-byte pieces per thread
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int n0 = blockIdx.x * (16 * WAVES) + wave * 16;
    int ks = blockIdx.y * k_per_split;
    int ke = min(k, ks + k_per_split);
    int n_chunks = (ke - ks + GS_KC - 1) / GS_KC;
    const bf16_t* wsafe = w + (size_t)min(n0 + (lane & 15), n - 1) * ldw;
    const bf16_t* wbase = wsafe + (lane >> 4) * 8;
    u32x4_t wcur[8], wnext[8], xr[XCHUNKS];
    f32x4_t acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Blocks start their K loop at different chunks and wrap around: row strides are often a
    // power of two, and blocks that all read the same K window at once would queue up on a few
    // memory channels.
    int rot = (blockIdx.x * 5 + blockIdx.y * 3) % n_chunks;
#define GS_CHUNK_BASE(c_) (ks + (((c_) + rot) >= n_chunks ? (c_) + rot - n_chunks : (c_) + rot) * GS_KC)
#define GS_LOAD_W(c_, dst_)                                                                     \
    {                                                                                           \
        int kb_ = GS_CHUNK_BASE(c_);                                                            \
        _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                         \
            bool in_ = kb_ + j * 32 + (lane >> 4) * 8 < ke;                                     \
            dst_[j] = *(const u32x4_t*)(in_ ? wbase + kb_ + j * 32 : wsafe);                    \
        }                                                                                       \
    }
#define GS_LOAD_X(c_)                                                                           \
    {                                                                                           \
        int kb_ = GS_CHUNK_BASE(c_);                                                            \
        _Pragma("unroll") for (int i = 0; i < XCHUNKS; ++i) {                                   \
            int piece_ = tid + i * THREADS;                                                  \
            int row_ = piece_ / (GS_KC / 8), gk_ = kb_ + (piece_ % (GS_KC / 8)) * 8;            \
            xr[i] = *(const u32x4_t*)(gk_ < ke ? x + (size_t)min(row_, m - 1) * ldx + gk_ : x); \
        }                                                                                       \
    }
#define GS_STORE_X(c_, buf_)                                                                    \
    {                                                                                           \
        int kb_ = GS_CHUNK_BASE(c_);                                                            \
        u32x4_t* sx_ = gs_smem + (buf_) * ROWS * GS_ROW;                                        \
        const u32x4_t zero_ = {0u, 0u, 0u, 0u};                                                 \
        _Pragma("unroll") for (int i = 0; i < XCHUNKS; ++i) {                                   \
            int piece_ = tid + i * THREADS;                                                  \
            int kc_ = piece_ % (GS_KC / 8);                                                     \
            sx_[(piece_ / (GS_KC / 8)) * GS_ROW + kc_] = kb_ + kc_ * 8 < ke ? xr[i] : zero_;    \
        }                                                                                       \
    }

    GS_LOAD_W(0, wcur)
    GS_LOAD_X(0)
    GS_STORE_X(0, 0)
    __syncthreads();
    for (int c = 0; c < n_chunks; ++c) {
        int buf = c & 1;
        bool more = c + 1 < n_chunks;
        if (more) {
            GS_LOAD_W(c + 1, wnext)
            GS_LOAD_X(c + 1)
        }
        const u32x4_t* sx = gs_smem + buf * ROWS * GS_ROW;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            bf16x8_t a = as_frag4(wcur[j]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                bf16x8_t b = as_frag4(sx[(mt * 16 + (lane & 15)) * GS_ROW + j * 4 + (lane >> 4)]);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
            }
        }
        if (more) {
            GS_STORE_X(c + 1, buf ^ 1)
#pragma unroll
            for (int j = 0; j < 8; ++j) wcur[j] = wnext[j];
        }
        __syncthreads();
    }
#undef GS_CHUNK_BASE
#undef GS_LOAD_W
#undef GS_LOAD_X
#undef GS_STORE_X
    // Accumulator element e of a lane: weight row (lane/16)*4 + e, activation row lane%16.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int gm = mt * 16 + (lane & 15);
        if (gm >= m) continue;
        if (EPI == EPI_SWIGLU && !PARTIAL) {
            // a lane holds weight rows 4g .. 4g+3 = two (gate, up) pairs
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
                int gn = n0 + (lane >> 4) * 4 + e;
                if (gn + 1 < n)
                    ((bf16_t*)out)[(size_t)gm * ldo + (gn >> 1)] = f32_to_bf16(silu_mul(acc[mt][e], acc[mt][e + 1]));
            }
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            int gn = n0 + (lane >> 4) * 4 + e;
            if (gn >= n) continue;
            if (PARTIAL) ((float*)out)[((size_t)blockIdx.y * m + gm) * n + gn] = acc[mt][e];
            else epilogue_store<EPI>(out, (size_t)gm * ldo + gn, acc[mt][e]);
        }
    }
}

// ---- at most 16 rows -------------------------------------------------------------------------
// The decode step of a small batch.  A block owns 16 weight rows and a K range; its four waves
// take a quarter of the range each and never meet before the end: weights and activations go
// from global memory (the activations are small and stay in L2) straight into MFMA operand
// registers, two rounds of 8 loads of 16 bytes per lane in flight, no LDS and no barrier in the
// loop.  With 16 rows per block even the widest projection gives thousands of waves, which is
// what keeps enough bytes in flight to stream weights at memory speed.  The four partial tiles
// are added in wave order through LDS, then comes the epilogue (or the split-K partial store).
constexpr int GK_KC = 256, GK_THREADS = 256;

template <int EPI, bool PARTIAL>
__global__ void __launch_bounds__(GK_THREADS)
gemm_kpar_kernel(const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw,
                 void* __restrict__ out, int ldo, int m, int n, int k, int k_per_split) {
    __shared__ float red[4][64][4];
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int g = lane >> 4, col = lane & 15;
    int tile = blockIdx.x, split = blockIdx.y;
    int bs = split * k_per_split, be = min(k, bs + k_per_split);
    int quarter = (((be - bs + 3) / 4) + 31) / 32 * 32;
    int ks = min(be, bs + wave * quarter), ke = min(be, ks + quarter);
    bool xok = col < m;
    const bf16_t* wsafe = w + (size_t)min(tile * 16 + col, n - 1) * ldw;
    const bf16_t* xsafe = x + (size_t)min(col, m - 1) * ldx;
    const bf16_t* wp = wsafe + g * 8;
    const bf16_t* xp = xsafe + g * 8;
    u32x4_t wc[8], xc[8], wn[8], xn[8];
    f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // No select behind a load (see the few-rows kernel): clamped addresses, and the activations
    // of a piece beyond K are zeroed just before they are multiplied.
#define GK_LOAD(kb_, wd_, xd_)                                                \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                           \
        bool in_ = (kb_) + j * 32 + g * 8 < ke;                               \
        wd_[j] = *(const u32x4_t*)(in_ ? wp + (kb_) + j * 32 : wsafe);        \
        xd_[j] = *(const u32x4_t*)(in_ ? xp + (kb_) + j * 32 : xsafe);        \
    }
    if (ks < ke) GK_LOAD(ks, wc, xc)
    for (int kb = ks; kb < ke; kb += GK_KC) {
        bool more = kb + GK_KC < ke;
        if (more) GK_LOAD(kb + GK_KC, wn, xn)
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            u32x4_t xv = kb + j * 32 + g * 8 < ke ? xc[j] : zero;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag4(wc[j]), as_frag4(xv), acc, 0, 0, 0);
        }
        if (more) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                wc[j] = wn[j];
                xc[j] = xn[j];
            }
        }
    }
#undef GK_LOAD
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][lane][e] = acc[e];
    __syncthreads();
    if (wave != 0 || !xok) return;
    float sum[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[e] = ((red[0][lane][e] + red[1][lane][e]) + red[2][lane][e]) + red[3][lane][e];
    // element e of a lane: weight row 4g + e of the tile, activation row lane%16
    int gn0 = tile * 16 + g * 4;
    if (EPI == EPI_SWIGLU && !PARTIAL) {
#pragma unroll
        for (int e = 0; e < 4; e += 2)
            if (gn0 + e + 1 < n)
                ((bf16_t*)out)[(size_t)col * ldo + ((gn0 + e) >> 1)] = f32_to_bf16(silu_mul(sum[e], sum[e + 1]));
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        int gn = gn0 + e;
        if (gn >= n) continue;
        if (PARTIAL) ((float*)out)[((size_t)split * m + col) * n + gn] = sum[e];
        else epilogue_store<EPI>(out, (size_t)col * ldo + gn, sum[e]);
    }
}

// out[m][n] (+)= sum over splits, in split order.
template <int EPI>
__global__ void gemm_splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ out,
                                          int ldo, int m, int n, int splits) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)m * n) return;
    int gm = (int)(idx / n), gn = (int)(idx - (long long)gm * n);
    float s = 0.f;
    size_t stride = (size_t)m * n;
    int i = 0;
    for (; i + 4 <= splits; i += 4) {      // four loads in flight, added in split order
        float a0 = partial[i * stride + idx], a1 = partial[(i + 1) * stride + idx];
        float a2 = partial[(i + 2) * stride + idx], a3 = partial[(i + 3) * stride + idx];
        s += a0;
        s += a1;
        s += a2;
        s += a3;
    }
    for (; i < splits; ++i) s += partial[i * stride + idx];
    epilogue_store<EPI>(out, (size_t)gm * ldo + gn, s);
}
