// bfloat16 matrix products on the gfx950 matrix cores: out[M,N] (+)= X[M,K] * W[N,K]^T with
// 32-bit accumulation.  Both operands are K-contiguous, which is what an MFMA lane wants: 8
// consecutive K values (16 bytes) of one row.
//
// Kernels:
//  * gemm_mfma_kernel, many rows (prefill): an output tile per block, each wave a grid of
//    v_mfma_f32_32x32x16_bf16 tiles (128x64 per wave in the 256-wide shapes, 64x64 in the
//    128x128 one); K staged 64 at a time through double-buffered LDS with one barrier per stage;
//    rows padded by 16 bytes so that 128-bit LDS reads of 16 rows fall into 16 different bank
//    groups.  The idea of the tiling (big tile per block, a grid of fragments per wave, padded
//    double-buffered LDS) is the reference's WMMA kernel
//    (rocml-kernels/kernels/gemm_xwt_wmma_impl.h:211-378); layouts, sizes and the instruction
//    schedule are for wave64 MFMA.  Blocks are renumbered so that each of the 8 XCDs works on a
//    contiguous range of tiles and its L2 sees few weight panels.
//  * gemm_skinny_kernel, few rows (decode, M <= 64): memory-bound; a block owns 16 weight rows
//    per wave and a K range.  Weights go straight from global memory into MFMA operand
//    registers (v_mfma_f32_16x16x32_bf16), 8 loads of 16 bytes in flight per lane; the
//    activations of the K range are shared through LDS.  Split-K partial sums go to a
//    workspace and are added in split order by a second kernel (or by the caller's next
//    kernel), so results do not depend on timing
//    (rocml-kernels/kernels/gemm_splitk_reduce.hip:4-10 has the same rule).
//    gemm_skinny_ahead_kernel is the same with weights and activations requested two steps
//    ahead and any number of waves a block from 2 to 16: for 17 to 64 rows, for the gated
//    product at every number of rows up to 64 (it cannot be cut along K, so the waves a block
//    are what makes its blocks one round over the CUs), and for products cut along K whose
//    blocks the host chose for the busiest CU.
//  * gemm_kpar_kernel, one or two rows: the waves of a block split K and meet once in LDS.
//  * gemm_residual_prescale_kernel, up to 16 rows: whole sums into the residual stream and the
//    next norm's operand in one pass.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // 16 bytes as a native vector: a
// conditional between two of these is a register select, between two uint4 structs it goes
// through memory and drags whole arrays into scratch

__device__ __forceinline__ bf16x8_t as_frag4(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

// EPI_SWIGLU: weight rows come in pairs (gate_j, up_j); the output is bfloat16 [M, N/2] with
// out[m][j] = silu(gate) * up (rocml-kernels/kernels/silu_mul.hip:12-20), formed from the 32-bit
// accumulators so that gate and up are never rounded or written.
enum GemmEpilogue : int { EPI_F32 = 0, EPI_BF16 = 1, EPI_ACC = 2, EPI_SWIGLU = 3 };

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// The scale of a norm whose product-side half was done by the producer of the residual stream
// (gemm_residual_prescale_kernel): the operand is bfloat16(x * gain), and the sums of this product
// still lack the factor 1 / sqrt(sum of x^2 / width + eps) of their row, which is formed here from
// the sums of squares per 16 columns that the producer left.  ssq null: nothing to scale.
struct RowScale { const float* ssq; int parts; float eps; float inv_width; };

// The scale of activation row lane%16 (the row an MFMA lane's sums belong to), the same in the
// four lanes of a row; rows beyond M get 1.  In two steps: row_scale_request (the whole wave works
// on every row: a lane loads a sixteenth or less of the row's sums, all rows' loads go out
// together, one trip to memory) and row_scale_finish (the lanes' sums meet by butterfly, in the
// same order whatever the row).
__device__ __forceinline__ void row_scale_request(RowScale rs, int lane, int m, float (&part)[16]) {
#pragma unroll
    for (int r = 0; r < 16; ++r) part[r] = 0.f;
    if (!rs.ssq) return;
    // No branch between the loads of different rows (a branch would make every row wait for its own
    // trip): rows beyond M read the last row again, lanes beyond the row's end read its start, and
    // what they read is not counted.
    if ((rs.parts & 3) == 0) {
        int chunks = rs.parts / 4;
        const float4* all = (const float4*)rs.ssq;
        for (int base = 0; base < chunks; base += 64) {
            bool ok = base + lane < chunks;
            int c = ok ? base + lane : 0;
            float4 v[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] = all[(size_t)min(r, m - 1) * chunks + c];
#pragma unroll
            for (int r = 0; r < 16; ++r) part[r] += ok ? (v[r].x + v[r].y) + (v[r].z + v[r].w) : 0.f;
        }
    } else {
        for (int base = 0; base < rs.parts; base += 64) {
            bool ok = base + lane < rs.parts;
            int p = ok ? base + lane : 0;
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] = rs.ssq[(size_t)min(r, m - 1) * rs.parts + p];
#pragma unroll
            for (int r = 0; r < 16; ++r) part[r] += ok ? v[r] : 0.f;
        }
    }
}

// red: 16 x RS_RED_STRIDE floats of LDS that the calling wave has to itself.  The lanes' sums meet
// there: every lane leaves its sixteen partial sums, then adds up a quarter of the row lane%16 and
// two butterfly steps finish it (a butterfly per row would be 96 exchanges instead of 2).
constexpr int RS_RED_STRIDE = 68;     // 16-byte aligned rows whose banks are staggered

__device__ __forceinline__ float row_scale_finish(RowScale rs, int lane, int m, const float (&part)[16], float* red) {
    if (!rs.ssq) return 1.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) red[r * RS_RED_STRIDE + lane] = part[r];
    __builtin_amdgcn_wave_barrier();
    const float4* mine = (const float4*)(red + (lane & 15) * RS_RED_STRIDE + (lane >> 4) * 16);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float4 v = mine[j];
        s += (v.x + v.y) + (v.z + v.w);
    }
    s += __shfl_xor(s, 16, 64);
    s += __shfl_xor(s, 32, 64);
    return (lane & 15) < m ? 1.0f / sqrtf(s * rs.inv_width + rs.eps) : 1.0f;
}

// The same scales formed by several waves, each for NR rows of its own from row0 (4 or 8: fewer
// loads in flight per lane, for kernels whose registers are taken by weights on their way):
// scale_out[row0 .. row0 + NR) in LDS; red: NR x RS_RED_STRIDE floats that the wave has to itself.
template <int NR>
__device__ __forceinline__ void row_scale_rows(RowScale rs, int lane, int m, int row0, float* red, float* scale_out) {
    static_assert(NR == 4 || NR == 8, "four or eight rows a wave");
    if (!rs.ssq) {
        if (lane < NR) scale_out[row0 + lane] = 1.0f;
        return;
    }
    float part[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) part[i] = 0.f;
    // (no branch between the loads of different rows, as in row_scale_request)
    if ((rs.parts & 3) == 0) {
        int chunks = rs.parts / 4;
        const float4* all = (const float4*)rs.ssq;
        for (int base = 0; base < chunks; base += 64) {
            bool ok = base + lane < chunks;
            int c = ok ? base + lane : 0;
            float4 v[NR];
#pragma unroll
            for (int i = 0; i < NR; ++i) v[i] = all[(size_t)min(row0 + i, m - 1) * chunks + c];
#pragma unroll
            for (int i = 0; i < NR; ++i) part[i] += ok ? (v[i].x + v[i].y) + (v[i].z + v[i].w) : 0.f;
        }
    } else {
        for (int base = 0; base < rs.parts; base += 64) {
            bool ok = base + lane < rs.parts;
            int p = ok ? base + lane : 0;
            float v[NR];
#pragma unroll
            for (int i = 0; i < NR; ++i) v[i] = rs.ssq[(size_t)min(row0 + i, m - 1) * rs.parts + p];
#pragma unroll
            for (int i = 0; i < NR; ++i) part[i] += ok ? v[i] : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < NR; ++i) red[i * RS_RED_STRIDE + lane] = part[i];
    __builtin_amdgcn_wave_barrier();
    constexpr int LPR = 64 / NR;                      // lanes that share a row, NR values each
    int i = lane / LPR, sub = lane % LPR;
    const float4* mine = (const float4*)(red + i * RS_RED_STRIDE + sub * NR);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NR / 4; ++j) {
        float4 v = mine[j];
        s += (v.x + v.y) + (v.z + v.w);
    }
#pragma unroll
    for (int off = 1; off < LPR; off <<= 1) s += __shfl_xor(s, off, 64);
    if (sub == 0) scale_out[row0 + i] = row0 + i < m ? 1.0f / sqrtf(s * rs.inv_width + rs.eps) : 1.0f;
}

template <int EPI>
__device__ __forceinline__ void epilogue_store(void* out, size_t idx, float v) {
    if (EPI == EPI_F32) ((float*)out)[idx] = v;
    else if (EPI == EPI_BF16) ((bf16_t*)out)[idx] = f32_to_bf16(v);
    else if (EPI == EPI_ACC) ((float*)out)[idx] += v;
}

// ---- many rows ---------------------------------------------------------------------------
// One kernel, two shapes (see GemmTile below): 256x256 with eight waves (two per SIMD, each
// 128x64) for products wide enough to give every CU such a tile, 128x128 with four waves of
// 64x64 (two blocks per CU) for the rest.  (256x128 with four waves of 128x64 was tried: one
// wave per SIMD has nobody to cover for it while it waits for weights from HBM.  Reading four
// bytes of every row's line some stages ahead, to pull it into L2, was tried too: the extra
// requests cost more than the earlier arrival gains, also when only one block of every tile
// column (for the weights) and one column in four (for the activations) does it.  Loading the operands straight into LDS
// (global_load_lds_dwordx4, K staged 32 at a time in five unpadded, XOR-swizzled buffers) was
// tried as well and gave the same results about 7% slower: a barrier every 16 products per wave,
// and the compiler answers such loads with a full wait on the LDS counter before the first
// product of every stage.)
constexpr int GM_BK = 64;
constexpr int GM_BAND = 8;                             // tile rows of a band (see the kernel)
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
using GemmTile256 = GemmTile<2, 4, 4, 2>;       // eight waves (two per SIMD), 128x64 each
using GemmTile192 = GemmTile<4, 2, 2, 3>;       // 256 rows x 192 columns, eight waves of 64x96

// Accumulator element e of a lane: row 8*(e/4) + 4*(lane/32) + e%4, column lane%32.
template <int EPI, typename T>
__device__ __forceinline__ void tile_epilogue(f32x16_t (&acc)[T::TM][T::TN], void* out, int ldo, int m, int n,
                                              int m0, int n0, int wm, int wn, int lane) {
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
            int gn = n0 + (wn * T::TN + j) * 32 + (lane & 31);
            if (EPI == EPI_SWIGLU) {
                // Neighbouring lanes hold neighbouring columns: the even one the gate, the odd one
                // the up value of one output column.  Of two neighbouring rows the even lane
                // finishes the first and the odd lane the second: one exchange per pair of rows,
                // and every lane has half of the exponentials and stores.
                bool odd = lane & 1;
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    float first = acc[i][j][e], second = acc[i][j][e + 1];
                    float got = __shfl_xor(odd ? first : second, 1, 64);    // even: up of row e; odd: gate of row e+1
                    float gate = odd ? got : first, up = odd ? second : got;
                    int gm = m0 + (wm * T::TM + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3) + (odd ? 1 : 0);
                    if (gm < m && (gn | 1) < n)
                        ((bf16_t*)out)[(size_t)gm * ldo + (gn >> 1)] = f32_to_bf16(silu_mul(gate, up));
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int gm = m0 + (wm * T::TM + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (gm < m && gn < n) epilogue_store<EPI>(out, (size_t)gm * ldo + gn, acc[i][j][e]);
            }
        }
}

template <int EPI, typename T>
__global__ void __launch_bounds__(T::THREADS)
gemm_mfma_kernel(const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw,
                 void* __restrict__ out, int ldo, int m, int n, int k, int tiles_m, int n_tiles,
                 int k_per_split, long long split_stride) {
    // With split_stride != 0 the K range is cut into pieces of k_per_split; piece p of a tile is
    // the work of block p * n_tiles + tile and goes, as 32-bit partial sums, to
    // out + p * split_stride (the caller instantiates the 32-bit store for that).
    extern __shared__ u32x4_t gm_smem[];              // [2 stages][A: BM rows | B: BN rows][GM_ROW]
    constexpr int STAGE = (T::BM + T::BN) * GM_ROW;
    constexpr int NREG = T::PA + T::PB;               // 16-byte pieces a thread moves per K stage
    constexpr int PROD = T::TM * T::TN;               // products per 16-wide K slice
    constexpr int KK = GM_BK / 16;                    // slices per stage
    static_assert(KK == 4, "the schedule below is written for four slices per stage");
    // piece r is stored after product r * SPAN / NREG of the first three slices (SPAN products);
    // its register is refilled one product later when every store has a free product behind it,
    // else right behind the store
    constexpr int SPAN = 3 * PROD;
    static_assert(SPAN >= NREG, "the stores must fit into the first three slices");
    constexpr bool REFILL_LATER = SPAN >= 2 * NREG;
    int per_xcd = gridDim.x / 8;
    int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    int split = logical / n_tiles;
    logical -= split * n_tiles;
    int ks = split * k_per_split;
    if (ks >= k) return;
    k = min(k - ks, k_per_split);                     // from here on: this block's K range, starting at 0
    x += ks;
    w += ks;
    out = (float*)out + split * split_stride;
    // Tiles are walked in bands of eight tile rows, down the band's columns: the 32 blocks that an
    // XCD holds at a time are then eight tile rows by four tile columns (twelve operand strips
    // through its L2 for 32 tiles) and not 32 rows of one column (33 strips), whatever the number of rows.
    int band_tiles = GM_BAND * (n_tiles / tiles_m), band = logical / band_tiles, in_band = logical - band * band_tiles;
    int band_rows = min(GM_BAND, tiles_m - band * GM_BAND);
    int m0 = (band * GM_BAND + in_band % band_rows) * T::BM, n0 = (in_band / band_rows) * T::BN;
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    int lrow = tid >> 3, lkc = tid & 7;
    int nk = (k + GM_BK - 1) / GM_BK;
    f32x16_t acc[T::TM][T::TN];
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // Schedule of one K stage (64 wide = four slices of 16), written out by hand and pinned with
    // scheduling barriers, because left alone the compiler sinks every LDS read to its first use
    // and gathers the stores behind the products:
    //  * the operand pieces of the next slice are read from LDS before the products of the
    //    current slice are issued (two register sets);
    //  * the pieces of the next stage, loaded from global memory one stage ago, are stored to the
    //    other LDS buffer between the products of slices 0 to 2 (evenly: LDS takes a 128-bit
    //    store at a quarter of the rate of a read, and bunched stores hold up the operand reads
    //    behind them), and each register is refilled from the stage after that: the memory pipes
    //    work while the matrix core does, and a load has a whole stage to arrive;
    //  * the one barrier of a stage stands after slice 2.  By then every wave has stored its
    //    pieces of the next stage and has read the last pieces of this one, so during slice 3 the
    //    first operands of the next stage are fetched and the matrix core does not wait for LDS
    //    when the stage changes.
    // Loads go to clamped addresses and are used as they come: rows beyond M or N only feed
    // outputs that are never stored, and a piece beyond K is zeroed when it is stored to LDS.
    // Nothing in the loop is conditional, so the count of outstanding loads is known at every
    // wait; the last stages load and store pieces nobody reads.
    u32x4_t reg[NREG];
    const bf16_t* src[NREG];
    int dst[NREG];                                    // LDS index of the piece within a stage
#pragma unroll
    for (int r = 0; r < NREG; ++r) {
        bool is_a = r < T::PA;
        int row = lrow + T::PASS_ROWS * (is_a ? r : r - T::PA);
        src[r] = is_a ? x + (size_t)min(m0 + row, m - 1) * ldx + lkc * 8
                      : w + (size_t)min(n0 + row, n - 1) * ldw + lkc * 8;
        dst[r] = (is_a ? 0 : T::BM * GM_ROW) + row * GM_ROW + lkc;
    }
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    int fa = (wm * T::TM * 32 + (lane & 31)) * GM_ROW + (lane >> 5);
    int fb = T::BM * GM_ROW + (wn * T::TN * 32 + (lane & 31)) * GM_ROW + (lane >> 5);
    // offset of this thread's piece in stage kt, or back to the row's start when it is beyond K
#define GM_KOFF(kt_) ((kt_) * GM_BK + lkc * 8 < k ? (kt_) * GM_BK : -lkc * 8)
    {
        int o0 = GM_KOFF(0);
        bool in0 = lkc * 8 < k;
#pragma unroll
        for (int r = 0; r < NREG; ++r) reg[r] = *(const u32x4_t*)(src[r] + o0);
#pragma unroll
        for (int r = 0; r < NREG; ++r) gm_smem[dst[r]] = in0 ? reg[r] : zero;
        int o1 = GM_KOFF(1);
#pragma unroll
        for (int r = 0; r < NREG; ++r) reg[r] = *(const u32x4_t*)(src[r] + o1);
    }
    __syncthreads();
    bf16x8_t a[2][T::TM], b[2][T::TN];
#pragma unroll
    for (int i = 0; i < T::TM; ++i) a[0][i] = as_frag4(gm_smem[fa + i * 32 * GM_ROW]);
#pragma unroll
    for (int j = 0; j < T::TN; ++j) b[0][j] = as_frag4(gm_smem[fb + j * 32 * GM_ROW]);
    for (int kt = 0; kt < nk; ++kt) {
        const u32x4_t* cur = gm_smem + (kt & 1) * STAGE;
        u32x4_t* nxt = gm_smem + ((kt + 1) & 1) * STAGE;
        bool in1 = (kt + 1) * GM_BK + lkc * 8 < k;    // is the piece held in registers inside K
        int o2 = GM_KOFF(kt + 2);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            int c = kk & 1;
            const u32x4_t* from = kk + 1 < KK ? cur + (kk + 1) * 2 : nxt;   // slice 3 fetches the next stage's slice 0
#pragma unroll
            for (int i = 0; i < T::TM; ++i) a[c ^ 1][i] = as_frag4(from[fa + i * 32 * GM_ROW]);
#pragma unroll
            for (int j = 0; j < T::TN; ++j) b[c ^ 1][j] = as_frag4(from[fb + j * 32 * GM_ROW]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < PROD; ++q) {
                acc[q / T::TN][q % T::TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    a[c][q / T::TN], b[c][q % T::TN], acc[q / T::TN][q % T::TN], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                // the piece whose place is product s of the stage: r with r * SPAN / NREG == s
                int slot = kk * PROD + q;
                int r = (slot * NREG + SPAN - 1) / SPAN;
                bool here = kk < 3 && r < NREG && r * SPAN / NREG == slot;
                int rp = ((slot - 1) * NREG + SPAN - 1) / SPAN;      // the piece one product earlier
                bool before = slot >= 1 && slot - 1 < SPAN && rp < NREG && rp * SPAN / NREG == slot - 1;
                if (here) {
                    nxt[dst[r]] = in1 ? reg[r] : zero;
                    if (!REFILL_LATER) reg[r] = *(const u32x4_t*)(src[r] + o2);
                } else if (REFILL_LATER && before) {
                    reg[rp] = *(const u32x4_t*)(src[rp] + o2);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kk == 2) __syncthreads();
        }
    }
#undef GM_KOFF
    tile_epilogue<EPI, T>(acc, out, ldo, m, n, m0, n0, wm, wn, lane);
}

// ---- few rows ----------------------------------------------------------------------------
constexpr int GS_KC = 256;                            // K values per chunk
constexpr int GS_ROW = GS_KC / 8 + 1;                 // uint4 per LDS row of activations

// Accumulator element e of a lane: weight row (lane/16)*4 + e, activation row lane%16.
template <int MT, int EPI, bool PARTIAL>
__device__ __forceinline__ void skinny_epilogue(const f32x4_t (&acc)[MT], void* out, int ldo, int m, int n, int n0,
                                                int lane, int split, float row_scale = 1.0f) {
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
                    ((bf16_t*)out)[(size_t)gm * ldo + (gn >> 1)] =
                        f32_to_bf16(silu_mul(acc[mt][e] * row_scale, acc[mt][e + 1] * row_scale));
            }
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            int gn = n0 + (lane >> 4) * 4 + e;
            if (gn >= n) continue;
            if (PARTIAL) ((float*)out)[((size_t)split * m + gm) * n + gn] = acc[mt][e];
            else epilogue_store<EPI>(out, (size_t)gm * ldo + gn, acc[mt][e]);
        }
    }
}

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
    skinny_epilogue<MT, EPI, PARTIAL>(acc, out, ldo, m, n, n0, lane, blockIdx.y);
}

// The same product for 17 to 64 rows.  With more rows a step costs more (four products and four
// LDS reads per weight fragment at 64 rows) and the chip holds fewer waves, so what a step waits
// for decides: here nothing in the loop waits for a load younger than a whole step.  The weights
// of step c+2 are requested when the products of step c have been issued (into the registers
// these have just read), the activations of step c+2 at the start of step c, and they are
// written to the other LDS buffer at the end of step c+1.  (Everything requested before the
// first product, four steps deep, was measured too: the waves then sit in the issue queue until
// the data has all but arrived.)
// All loads are buffer loads: the hardware returns zeros for an offset beyond the buffer, which
// takes the place of every clamp and branch (rows beyond N or M, pieces beyond the K range,
// whole steps beyond the last) and leaves the compiler's wait counts exact; a lane's address is
// one 32-bit register for all of its loads.  A block's weight rows are its buffer, so only the
// bytes of 16 * WAVES rows must fit 31 bits.
constexpr uint32_t GA_NOWHERE = 0x80000000u;         // an offset beyond any buffer here

__device__ __forceinline__ __amdgpu_buffer_rsrc_t ga_buffer(const void* base, long long bytes) {
    // raw buffer (stride 0), 32-bit data format; the range check is on the byte offset
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)min(bytes, (long long)0x7fffffff), 0x00020000);
}

template <int MT, int EPI, bool PARTIAL, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
gemm_skinny_ahead_kernel(const bf16_t* x, int ldx, const bf16_t* w, int ldw, void* out, int ldo, int m, int n,
                         int k, int k_per_split, RowScale rs = RowScale{}) {
    extern __shared__ u32x4_t gs_smem[];              // [2][MT*16][GS_ROW]
    constexpr int ROWS = MT * 16;
    constexpr int THREADS = 64 * WAVES;
    constexpr int XPIECES = ROWS * (GS_KC / 8);       // 16-byte pieces of the activations per step
    constexpr int XL = (XPIECES + THREADS - 1) / THREADS;   // loads per thread and step
    constexpr bool XEXACT = XPIECES % THREADS == 0;   // else the last round has threads without a piece
    constexpr int D = 2;                              // steps that the weights are requested ahead
    int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int block_row = blockIdx.x * (16 * WAVES);
    int n0 = block_row + wave * 16;
    int ks = blockIdx.y * k_per_split;
    int ke = min(k, ks + k_per_split);
    int n_steps = (ke - ks + GS_KC - 1) / GS_KC;
    int rows_here = min(16 * WAVES, n - block_row);
    __amdgpu_buffer_rsrc_t wbuf = ga_buffer(w + (size_t)block_row * ldw, ((long long)(rows_here - 1) * ldw + k) * 2);
    __amdgpu_buffer_rsrc_t xbuf = ga_buffer(x, ((long long)(m - 1) * ldx + k) * 2);
    // byte offsets of a lane's first piece: weight row lane%16 of the wave's tile, K piece lane/16
    uint32_t woff = ((uint32_t)(wave * 16 + (lane & 15)) * (uint32_t)ldw + (lane >> 4) * 8) * 2;
    uint32_t xoff[XL];
    int xk[XL];                                       // K offset of activation piece i within a step
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        int piece = tid + i * THREADS;
        xk[i] = (piece % (GS_KC / 8)) * 8;
        xoff[i] = ((uint32_t)(piece / (GS_KC / 8)) * (uint32_t)ldx + xk[i]) * 2;
        if (!XEXACT && piece >= XPIECES) xk[i] = 0x40000000;     // beyond every K range: never loaded
    }
    u32x4_t wr[D][8], xr[2][XL];
    f32x4_t acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Blocks start their K loop at different steps and wrap around: row strides are often a
    // power of two, and blocks that all read the same K window at once would queue up on a few
    // memory channels.
    int rot = (blockIdx.x * 5 + blockIdx.y * 3) % n_steps;
#define GA_BASE(c_) (ks + (((c_) + rot) >= n_steps ? (c_) + rot - n_steps : (c_) + rot) * GS_KC)
    // (neither the optimizer nor the scheduler may move a load across this)
#define GA_KEEP_ORDER asm volatile("" ::: "memory"); __builtin_amdgcn_sched_barrier(0);
    // (weights beyond the K range are not multiplied by zero but not loaded: a row's stride may
    // be longer than K, and what lies between is anything)
#define GA_LOAD_W(c_, set_)                                                                     \
    {                                                                                           \
        int kb_ = GA_BASE(c_);                                                                  \
        bool step_ = (c_) < n_steps;                                                            \
        _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                         \
            bool in_ = step_ && kb_ + j * 32 + (lane >> 4) * 8 < ke;                            \
            wr[set_][j] = __builtin_amdgcn_raw_buffer_load_b128(                                \
                wbuf, in_ ? woff + (uint32_t)kb_ * 2 + j * 64 : GA_NOWHERE, 0, 0);              \
        }                                                                                       \
    }
#define GA_LOAD_X(c_, set_)                                                                     \
    {                                                                                           \
        int kb_ = GA_BASE(c_);                                                                  \
        bool step_ = (c_) < n_steps;                                                            \
        _Pragma("unroll") for (int i = 0; i < XL; ++i) {                                        \
            bool in_ = step_ && kb_ + xk[i] < ke;                                               \
            xr[set_][i] = __builtin_amdgcn_raw_buffer_load_b128(                                \
                xbuf, in_ ? xoff[i] + (uint32_t)kb_ * 2 : GA_NOWHERE, 0, 0);                    \
        }                                                                                       \
    }
    // step c lives in register set and LDS buffer c % 2
#define GA_STORE_X(set_)                                                                        \
    {                                                                                           \
        u32x4_t* sx_ = gs_smem + (set_) * ROWS * GS_ROW;                                        \
        _Pragma("unroll") for (int i = 0; i < XL; ++i) {                                        \
            int piece_ = tid + i * THREADS;                                                     \
            if (XEXACT || piece_ < XPIECES)                                                     \
                sx_[(piece_ / (GS_KC / 8)) * GS_ROW + piece_ % (GS_KC / 8)] = xr[set_][i];      \
        }                                                                                       \
    }
    GA_LOAD_X(0, 0)
    GA_KEEP_ORDER
    GA_LOAD_W(0, 0)
    GA_KEEP_ORDER
    GA_LOAD_X(1, 1)
    GA_KEEP_ORDER
    GA_LOAD_W(1, 1)
    GA_KEEP_ORDER
    // The rows' scales, if the operand lacks them (the gated epilogue of at most 16 rows applies
    // them): the block's first waves form them, four rows each, while the first weights are on
    // their way and leave them in LDS for the epilogue.
    constexpr bool SCALES = MT == 1 && EPI == EPI_SWIGLU && !PARTIAL;
    __shared__ float ga_scale[16];
    __shared__ __attribute__((aligned(16))) float ga_red[SCALES ? 16 * RS_RED_STRIDE : 4];
    constexpr int SCALE_WAVES = WAVES >= 4 ? 4 : 2, SCALE_ROWS = 16 / SCALE_WAVES;
    if (SCALES && wave < SCALE_WAVES)
        row_scale_rows<SCALE_ROWS>(rs, lane, m, wave * SCALE_ROWS, ga_red + wave * SCALE_ROWS * RS_RED_STRIDE, ga_scale);
    GA_STORE_X(0)
    __syncthreads();
    for (int c0 = 0; c0 < n_steps; c0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            int c = c0 + u;
            if (c >= n_steps) break;
            // the activations of step c+2 take the registers that step c's were stored from
            GA_LOAD_X(c + 2, u)
            GA_KEEP_ORDER
            const u32x4_t* sx = gs_smem + u * ROWS * GS_ROW;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                bf16x8_t a = as_frag4(wr[u][j]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    bf16x8_t b = as_frag4(sx[(mt * 16 + (lane & 15)) * GS_ROW + j * 4 + (lane >> 4)]);
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
                }
            }
            // (a product has no side effect and would be sunk below the loads that follow, which
            // then could not take the registers it reads: tie the sums to this place)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(acc[mt]));
            GA_KEEP_ORDER
            GA_LOAD_W(c + D, u)
            GA_KEEP_ORDER
            GA_STORE_X(u ^ 1)
            __syncthreads();
        }
    }
#undef GA_BASE
#undef GA_KEEP_ORDER
#undef GA_LOAD_W
#undef GA_LOAD_X
#undef GA_STORE_X
    float row_scale = SCALES ? ga_scale[lane & 15] : 1.0f;
    skinny_epilogue<MT, EPI, PARTIAL>(acc, out, ldo, m, n, n0, lane, blockIdx.y, row_scale);
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
                 void* __restrict__ out, int ldo, int m, int n, int k, int k_per_split, RowScale rs) {
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
    // (the rows' scales for the gated epilogue: formed by the last wave while its first loads are
    // on their way, handed to the first wave through LDS)
    constexpr bool SCALES = EPI == EPI_SWIGLU && !PARTIAL;
    __shared__ float gk_scale[16];
    __shared__ __attribute__((aligned(16))) float gk_red[SCALES ? 16 * RS_RED_STRIDE : 4];
    if (SCALES && wave == 3) {
        float scale_part[16];
        row_scale_request(rs, lane, m, scale_part);
        float mine = row_scale_finish(rs, lane, m, scale_part, gk_red);
        if (lane < 16) gk_scale[lane] = mine;
    }
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
    if (wave != 0) return;
    float row_scale = SCALES ? gk_scale[lane & 15] : 1.0f;
    if (!xok) return;
    float sum[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[e] = ((red[0][lane][e] + red[1][lane][e]) + red[2][lane][e]) + red[3][lane][e];
    // element e of a lane: weight row 4g + e of the tile, activation row lane%16
    int gn0 = tile * 16 + g * 4;
    if (EPI == EPI_SWIGLU && !PARTIAL) {
#pragma unroll
        for (int e = 0; e < 4; e += 2)
            if (gn0 + e + 1 < n)
                ((bf16_t*)out)[(size_t)col * ldo + ((gn0 + e) >> 1)] =
                    f32_to_bf16(silu_mul(sum[e] * row_scale, sum[e + 1] * row_scale));
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

// ---- at most 16 rows: the residual sum, and the next norm prepared ------------------------------
// resid[M, N] += X[M, K] * W[N, K]^T with whole sums (a block owns 16 weight rows and all of K; its
// waves split K and meet once in LDS, in wave order), and in the same pass what the norm that
// reads the residual stream next would otherwise need a kernel of its own for: xg = bfloat16(resid *
// gain), the operand of the next product up to the row's scale, and ssq[row][tile], the sum of
// squares of the block's 16 columns of the row.  Whoever consumes the next product's sums
// multiplies them by 1 / sqrt(sum of ssq[row] / N + eps): the norm's scale is one number per row
// and commutes with the product.  A decode step of a few sequences is priced by the kernels that
// follow one another, not by bytes; this takes two norms out of every layer.
template <int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
gemm_residual_prescale_kernel(const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw,
                              float* resid, int ldr, const float* __restrict__ gain, bf16_t* __restrict__ xg, int ldg,
                              float* __restrict__ ssq, int tiles, int m, int n, int k) {
    __shared__ float red[WAVES][64][4];
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int g = lane >> 4, col = lane & 15;
    int tile = blockIdx.x;
    int share = (((k + WAVES - 1) / WAVES) + 31) / 32 * 32;
    int ks = min(k, wave * share), ke = min(k, ks + share);
    const bf16_t* wsafe = w + (size_t)min(tile * 16 + col, n - 1) * ldw;
    const bf16_t* xsafe = x + (size_t)min(col, m - 1) * ldx;
    const bf16_t* wp = wsafe + g * 8;
    const bf16_t* xp = xsafe + g * 8;
    u32x4_t wc[8], xc[8], wn[8], xn[8];
    f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
    bool xrow = col < m;        // lanes of rows beyond M load no activations (their sums are not stored)
#pragma unroll
    for (int j = 0; j < 8; ++j) xc[j] = xn[j] = u32x4_t{0u, 0u, 0u, 0u};
    // (no select behind a load: clamped addresses; a piece beyond the wave's K range is zeroed on
    // the activation side just before it is multiplied)
#define GR_LOAD(kb_, wd_, xd_)                                                \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                           \
        bool in_ = (kb_) + j * 32 + g * 8 < ke;                               \
        wd_[j] = *(const u32x4_t*)(in_ ? wp + (kb_) + j * 32 : wsafe);        \
        if (xrow) xd_[j] = *(const u32x4_t*)(in_ ? xp + (kb_) + j * 32 : xsafe); \
    }
    if (ks < ke) GR_LOAD(ks, wc, xc)
    // The first wave finishes the block's outputs: what it needs of the residual stream and of the
    // gain is asked for now, so that it has arrived when the sums are ready.
    int n0 = tile * 16 + g * 4;
    bool row_ok = col < m;
    bool vec = row_ok && n0 + 3 < n && (ldr & 3) == 0 && (ldg & 3) == 0;
    float4 r_old = make_float4(0.f, 0.f, 0.f, 0.f), gn = r_old;
    if (wave == 0 && vec) {
        r_old = *(const float4*)(resid + (size_t)col * ldr + n0);
        gn = *(const float4*)(gain + n0);
        asm volatile("" ::: "memory");          // (the loads stay here)
    }
    for (int kb = ks; kb < ke; kb += GK_KC) {
        bool more = kb + GK_KC < ke;
        if (more) GR_LOAD(kb + GK_KC, wn, xn)
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
#undef GR_LOAD
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][lane][e] = acc[e];
    __syncthreads();
    if (wave != 0) return;
    // element e of a lane: weight row (output column) 16 tile + 4g + e, activation row lane%16
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float sum = red[0][lane][e];
#pragma unroll
        for (int wv = 1; wv < WAVES; ++wv) sum += red[wv][lane][e];
        v[e] = sum;
    }
    float ss = 0.f;
    if (vec) {
        float4 r = r_old;
        r.x += v[0]; r.y += v[1]; r.z += v[2]; r.w += v[3];
        *(float4*)(resid + (size_t)col * ldr + n0) = r;
        *(uint2*)(xg + (size_t)col * ldg + n0) = make_uint2(f32x2_to_bf16x2(r.x * gn.x, r.y * gn.y),
                                                             f32x2_to_bf16x2(r.z * gn.z, r.w * gn.w));
        ss = fmaf(r.x, r.x, fmaf(r.y, r.y, fmaf(r.z, r.z, r.w * r.w)));
    } else if (row_ok) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n0 + e >= n) continue;
            float r = resid[(size_t)col * ldr + n0 + e] + v[e];
            resid[(size_t)col * ldr + n0 + e] = r;
            xg[(size_t)col * ldg + n0 + e] = f32_to_bf16(r * gain[n0 + e]);
            ss = fmaf(r, r, ss);
        }
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (row_ok && g == 0) ssq[(size_t)col * tiles + tile] = ss;
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
