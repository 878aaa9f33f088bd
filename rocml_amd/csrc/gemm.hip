// Matrix products of the decoder: out[M,N] (+)= X[M,K] * W[N,K]^T, weights row-major
// [out, in] as the reference keeps them (rocml/src/weights/mod.rs:78-98).  bfloat16 operands
// go to the MFMA kernels when their layout allows 16-byte loads; everything else, and the
// whole 32-bit path, goes to the plain tiled kernel.
#include "common.h"
#include "gemm_tile.h"
#include "gemm_mfma.h"

ROCML_LAST_ERROR_FN(gemm)

enum GemmAlgo : int { ALGO_AUTO = 0, ALGO_PLAIN = 1, ALGO_MFMA_TILE = 2, ALGO_MFMA_SKINNY = 3, ALGO_MFMA_KPAR = 4,
                      ALGO_MFMA_TILE256 = 5, ALGO_MFMA_TILE192 = 6, ALGO_MFMA_TILE128X192 = 7, ALGO_MFMA_TILE256X96 = 8,
                      ALGO_MFMA_TILE64X256 = 9 };

static int round_up(int a, int b) { return (a + b - 1) / b * b; }

template <typename K>
static int allow_lds(K kernel, int bytes, const char* name) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess)
        return rocml_fail("%s: cannot reserve %d bytes of LDS: %s", name, bytes, hipGetErrorString(e));
    return 0;
}

struct SplitPlan { int defer; int* deferred; RowScale rs; int max_splits; };   // max_splits: the most K pieces the caller wants

template <int EPI, typename T>
static int launch_mfma_tile_as(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m,
                               int n, int k, int splits, void* workspace, SplitPlan plan, hipStream_t stream) {
    static bool ready = false;
    if (!ready) {
        if (allow_lds(gemm_mfma_kernel<EPI, T>, T::LDS_BYTES, "gemm")) return 1;
        if (allow_lds(gemm_mfma_kernel<EPI_F32, T>, T::LDS_BYTES, "gemm")) return 1;
        ready = true;
    }
    int tiles_m = ceil_div(m, T::BM), tiles_n = ceil_div(n, T::BN);
    int n_tiles = tiles_m * tiles_n;
    if (splits <= 1) {
        gemm_mfma_kernel<EPI, T><<<round_up(n_tiles, 8), T::THREADS, T::LDS_BYTES, stream>>>(
            (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, tiles_m, n_tiles, k, 0);
        return 0;
    }
    // K cut in pieces: 32-bit partial sums [piece][M][N] in the workspace, added in order by the
    // caller's next kernel or by the reduce kernel here
    int k_per_split = round_up(ceil_div(k, splits), GM_BK);
    splits = ceil_div(k, k_per_split);
    gemm_mfma_kernel<EPI_F32, T><<<round_up(n_tiles * splits, 8), T::THREADS, T::LDS_BYTES, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, workspace, n, m, n, k, tiles_m, n_tiles, k_per_split,
        (long long)m * n);
    if (plan.defer && ldo == n) {
        *plan.deferred = splits;
        return 0;
    }
    long long total = (long long)m * n;
    gemm_splitk_reduce_kernel<EPI><<<ceil_div(total, 256), 256, 0, stream>>>((const float*)workspace, out, ldo, m, n, splits);
    return 0;
}

// The tile shapes of the many-rows kernel, as rows x columns of a block's tile: 128x128 (four waves
// of 64x64, two blocks a CU), 256x256 (eight waves of 128x64), 256x192 (eight of 64x96), 128x192
// (four of 64x96), 256x96 (four of 64x96, the whole of up to 256 rows against a narrow strip of
// weights) and 64x256 (four of 64x64 side by side, for products of few rows).
using GemmTile128x192 = GemmTile<2, 2, 2, 3>;
using GemmTile256x96 = GemmTile<4, 1, 2, 3>;
using GemmTile64x256 = GemmTile<1, 4, 2, 2>;

// What a tile shape costs: microseconds per 64-wide K stage for a CU that holds as many blocks of it
// as fit (`cap`), when half the chip or less is at work (`light`) and when all of it is (`full`: the
// memory system is shared and the clock drops under load), and, for the shape of which two fit,
// for a CU that holds one alone.  Measured on the Qwen3-8B and 14B products at 80 to 8192 rows.
struct TileKind { int bm, bn, cap; double light, full, alone; int shape; };
static const TileKind TILE_KINDS[] = {
    {128, 128, 2, 1.21, 1.25, 0.88, 1}, {256, 256, 1, 1.55, 1.85, 0.0, 2}, {256, 192, 1, 1.22, 1.50, 0.0, 3},
    {128, 192, 1, 1.00, 1.04, 0.0, 4},  {256, 96, 1, 1.03, 1.12, 0.0, 5},  {64, 256, 1, 0.93, 1.05, 0.0, 6}};

// An estimate of a product's time in microseconds with tiles of `kind` and K cut into `pieces`
// (each piece the work of a block of its own, 32-bit partial sums written once here and read once
// by whoever adds them): the rounds of blocks the chip holds at a time, each round as long as its
// K stages at the rate of the CUs' load, but no shorter than the busiest CU needs to pull its
// blocks' operands (36 GB/s a CU: with few rows it is the weights' arrival that a block waits for,
// and more, smaller blocks pull more at a time); a fixed part for the launch; the bytes the
// epilogue moves; never less than the weights need to arrive at all.  The constants were fitted
// to measurements of 103 products (the Qwen3-8B, 14B and 0.6B shapes at 52 to 8192 rows, six tile
// shapes, one to eight pieces): the choice made on this estimate is 0.9 % behind the best choice
// on average and within 5 % for nine in ten.
static double tile_cost(const TileKind& kind, int pieces, int m, int n, int k, int epi, int cus) {
    long long tiles = (long long)ceil_div(m, kind.bm) * ceil_div(n, kind.bn);
    int k_per_piece = round_up(ceil_div(k, pieces), GM_BK);
    pieces = ceil_div(k, k_per_piece);
    long long blocks = tiles * pieces, slots = (long long)cus * kind.cap;
    double stages = (double)(k_per_piece / GM_BK);
    auto stage_us = [&](long long together) {          // blocks on the chip at the same time, at most `slots`
        double share = (double)together / (double)cus;
        if (kind.cap == 2 && together <= cus) return kind.alone * (1.0 + 0.2 * (share > 0.5 ? share - 0.5 : 0.0));
        double busy = (double)together / (double)slots;
        double w = busy <= 0.5 ? 0.0 : busy >= 1.0 ? 1.0 : (busy - 0.5) * 2.0;
        return kind.light + (kind.full - kind.light) * w;
    };
    long long rounds = blocks / slots, rest = blocks % slots;
    double t = (double)rounds * stages * stage_us(slots) + (rest ? stages * stage_us(rest) : 0.0);
    double pulled = (double)(kind.bn + (m < kind.bm ? m : kind.bm)) * k_per_piece * 2.0 * (double)ceil_div(blocks, (long long)cus);
    if (t < pulled / 36.0e3) t = pulled / 36.0e3;
    t += 3.0;
    double moved = epi == EPI_SWIGLU ? (double)m * n
                   : pieces > 1      ? (double)m * n * 4.0 * pieces
                                     : (double)m * n * 4.0 * (epi == EPI_ACC ? 2.0 : 1.0);
    t += moved / 2.0e6;
    double floor_us = (double)n * k * 2.0 / 5.5e6;                  // the weights at 5.5 TB/s
    if (t < floor_us) t = floor_us;
    if (pieces > 1) t += (double)pieces * m * n * 4.0 / 5.0e6;      // the partial sums read again
    return t;
}

// shape: 0 = choose, else a TileKind's number (then K stays whole).  The choice is the smallest
// estimate over shapes and pieces.  What counts is the CU with the most work: 6144 columns are 24
// tiles of 256, which with 2048 rows leave a quarter of the chip idle, or 32 tiles of 192, which
// fill it; a product of 256 rows and 24576 columns is 384 tiles of 128x128, one and a half to a
// CU, or 256 of 128x192, one each.  A product with few tiles (few rows, or a narrow output)
// leaves most CUs idle while a few walk through all of K: then K is cut into up to 8 pieces.
template <int EPI>
static int launch_mfma_tile(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m,
                            int n, int k, int shape, void* workspace, long long workspace_bytes, SplitPlan plan,
                            hipStream_t stream) {
    int splits = 1;
    const int cus = cu_count();
    if (shape == 0) {
        double best = 1e30;
        for (const auto& kind : TILE_KINDS) {
            for (int pieces = 1; pieces <= 8 && pieces <= plan.max_splits; ++pieces) {
                if (pieces > 1 && (EPI == EPI_SWIGLU || k / pieces < 256 || !workspace ||
                                   (long long)pieces * m * n * (long long)sizeof(float) > workspace_bytes))
                    break;
                double t = tile_cost(kind, pieces, m, n, k, EPI, cus);
                if (t < best) { best = t; shape = kind.shape; splits = pieces; }
            }
        }
    }
    switch (shape) {
        case 6: return launch_mfma_tile_as<EPI, GemmTile64x256>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
        case 5: return launch_mfma_tile_as<EPI, GemmTile256x96>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
        case 4: return launch_mfma_tile_as<EPI, GemmTile128x192>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
        case 3: return launch_mfma_tile_as<EPI, GemmTile192>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
        case 2: return launch_mfma_tile_as<EPI, GemmTile256>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
        default: return launch_mfma_tile_as<EPI, GemmTile128>(x, ldx, w, ldw, out, ldo, m, n, k, splits, workspace, plan, stream);
    }
}

// The two-steps-ahead kernel on a product that cannot be cut along K (the gated product), with
// WAVES waves a block, each on 16 columns.
template <int MT, int EPI, int WAVES>
static int launch_ahead_whole(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m, int n,
                              int k, RowScale rs, hipStream_t stream) {
    constexpr int LDS = 2 * MT * 16 * GS_ROW * 16;
    static bool ready = false;
    if (!ready) {
        if (allow_lds(gemm_skinny_ahead_kernel<MT, EPI, false, WAVES>, LDS, "gemm")) return 1;
        ready = true;
    }
    gemm_skinny_ahead_kernel<MT, EPI, false, WAVES><<<dim3(ceil_div(n, 16 * WAVES), 1), 64 * WAVES, LDS, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, round_up(k, GS_KC), rs);
    return 0;
}

// Waves a block for such a product.  A CU pulls weight rows in 64-byte runs at a limited rate (the
// kernel's loads put a row's four pieces into the lanes of one instruction) and a second block on
// a CU stages the activations again, so the blocks should be one round that uses every CU: the
// fewest waves whose blocks the chip holds at once.  Measured at 64 rows: 24576 columns in 44 us
// with six waves (256 blocks; eight waves are 192 blocks and leave a quarter of 256 CUs idle:
// 49 us; five are two rounds: 72), 34816 x 5120 in 79 us with nine (eight: 116), 51200 x 5120 in
// 115 us with sixteen (eight: 124).  ``skip_from..skip_to``: counts whose kernel does not fit its
// registers.  A product wider than one round of the largest blocks gets the count that leaves the
// fewest columns on the busiest CU.
static int ahead_waves(int n, int cus, int skip_from, int skip_to) {
    for (int waves = 2; waves <= 16; ++waves)
        if ((waves < skip_from || waves > skip_to) && ceil_div(n, 16 * waves) <= cus) return waves;
    int best = 16, best_cols = 1 << 30;
    for (int waves = 16; waves >= 2; --waves) {
        if (waves >= skip_from && waves <= skip_to) continue;
        int cols = ceil_div(ceil_div(n, 16 * waves), cus) * 16 * waves;
        if (cols < best_cols) {
            best = waves;
            best_cols = cols;
        }
    }
    return best;
}

// The same kernel on one K range of a product that is cut along K: 32-bit partial sums
// [split][M][N] into the workspace.
template <int MT, int WAVES>
static int launch_ahead_split(const void* x, int ldx, const void* w, int ldw, void* workspace, int m, int n, int k,
                              int splits, int k_per_split, hipStream_t stream) {
    constexpr int LDS = 2 * MT * 16 * GS_ROW * 16;
    static bool ready = false;
    if (!ready) {
        if (allow_lds(gemm_skinny_ahead_kernel<MT, EPI_F32, true, WAVES>, LDS, "gemm")) return 1;
        ready = true;
    }
    gemm_skinny_ahead_kernel<MT, EPI_F32, true, WAVES><<<dim3(ceil_div(n, 16 * WAVES), splits), 64 * WAVES, LDS, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, workspace, n, m, n, k, k_per_split);
    return 0;
}

// Blocks of a product that may be cut along K: waves a block (16 columns each) and K pieces, so
// that the CU with the most work has as little as possible: its weight bytes (rounds of blocks
// times a block's columns times its K range) plus its share of the partial sums, which are
// written once and read once.  6144 x 4096 at 8 rows: 64 blocks of six waves times four pieces are
// one round of 256 equal blocks; 96 blocks of four waves times four pieces leave half the CUs with
// two blocks and half with one.
struct BlockChoice { int waves, splits, k_per_split; };

// An estimate of the busiest CU's time in microseconds.  A wave keeps two steps of weights
// (16 KB) on their way for the two microseconds a trip takes, a CU pulls such rows at up to about
// 45 GB/s however many waves ask (measured: 2.9 us more per 16 columns x 4096 a CU), a block
// stages its rows' activations of its K range through LDS once, LDS holds so many blocks of these
// rows at a time, and the partial sums are written here and read by the next kernel.
static double block_cost(BlockChoice c, int m, int row_tiles, int n, int cus) {
    const double lds_block = 2.0 * row_tiles * 16 * GS_ROW * 16;
    const int resident = (int)(160.0 * 1024 / lds_block) < 1 ? 1 : (int)(160.0 * 1024 / lds_block);
    long long blocks = (long long)ceil_div(n, 16 * c.waves) * c.splits;
    int per_cu = (int)ceil_div(blocks, (long long)cus);
    int together = per_cu < resident ? per_cu : resident;
    double rounds = (double)ceil_div(per_cu, together);
    double rate = 8.0e3 * c.waves * together;                              // bytes per microsecond
    if (rate > 45.0e3) rate = 45.0e3;
    double weights = 16.0 * c.waves * c.k_per_split * 2.0 * together;      // of the blocks that run together
    double staged = 16.0 * row_tiles * c.k_per_split * 2.0 * together;
    double cost = rounds * (weights / rate + staged / 100.0e3 + 3.0);
    if (c.splits > 1) cost += (double)c.splits * (m * (double)n * 8.0 / 2.0e6 + 0.15);
    return cost;
}

static BlockChoice choose_blocks(BlockChoice usual, int m, int row_tiles, int n, int k, int cus,
                                 long long workspace_bytes, int skip_from, int skip_to, int max_splits) {
    // (a step asks for the same few products over and over: the last answers are kept)
    // (the answer depends on the usual blocks and on the skipped wave counts too, which differ
    // between the callers that share this table)
    struct Kept { int m, row_tiles, n, k, cus; long long workspace_bytes; BlockChoice usual; int skip_from, skip_to, max_splits;
                  BlockChoice choice; bool set; };
    static thread_local Kept kept[64];
    Kept& slot = kept[((unsigned)n * 31u + (unsigned)k * 7u + (unsigned)m) % 64u];
    if (slot.set && slot.m == m && slot.row_tiles == row_tiles && slot.n == n && slot.k == k && slot.cus == cus &&
        slot.workspace_bytes == workspace_bytes && slot.usual.waves == usual.waves && slot.usual.splits == usual.splits &&
        slot.usual.k_per_split == usual.k_per_split && slot.skip_from == skip_from && slot.skip_to == skip_to &&
        slot.max_splits == max_splits)
        return slot.choice;
    BlockChoice best = usual;
    double best_cost = 1e30;
    for (int kps = GS_KC; kps < k + GS_KC; kps += GS_KC) {
        int splits = ceil_div(k, kps);
        if (splits > max_splits) continue;
        if (splits > 1 && (kps < 2 * GS_KC || (long long)splits * m * n * (long long)sizeof(float) > workspace_bytes)) continue;
        for (int waves = 2; waves <= 16; ++waves) {
            if (waves >= skip_from && waves <= skip_to) continue;
            BlockChoice c{waves, splits, kps};
            double cost = block_cost(c, m, row_tiles, n, cus);
            if (cost < best_cost * 0.999) {
                best_cost = cost;
                best = c;
            }
        }
    }
    // the usual blocks (four or eight waves, about two blocks or one a CU) unless the estimate
    // promises a clear gain: it is rough, and they are what the kernels were tuned with
    BlockChoice choice = best_cost < 0.93 * block_cost(usual, m, row_tiles, n, cus) ? best : usual;
    slot = Kept{m, row_tiles, n, k, cus, workspace_bytes, usual, skip_from, skip_to, max_splits, choice, true};
    return choice;
}

template <int MT, int EPI>
static int launch_skinny(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m, int n,
                         int k, void* workspace, long long workspace_bytes, SplitPlan plan, hipStream_t stream) {
    const int cus = cu_count();
    if constexpr (EPI == EPI_SWIGLU) {
        // The gated epilogue needs whole sums: the kernel that requests two steps ahead, whatever
        // the number of rows, with the number of waves that makes its blocks one round.  (At 49 to
        // 64 rows the kernels of 13 to 15 waves need more registers than 832 to 960 threads
        // leave each.)
        switch (ahead_waves(n, cus, MT == 4 ? 13 : 17, MT == 4 ? 15 : 17)) {
#define AHEAD_CASE(W_) case W_: return launch_ahead_whole<MT, EPI, W_>(x, ldx, w, ldw, out, ldo, m, n, k, plan.rs, stream);
            AHEAD_CASE(2) AHEAD_CASE(3) AHEAD_CASE(4) AHEAD_CASE(5) AHEAD_CASE(6) AHEAD_CASE(7) AHEAD_CASE(8)
            AHEAD_CASE(9) AHEAD_CASE(10) AHEAD_CASE(11) AHEAD_CASE(12) AHEAD_CASE(13) AHEAD_CASE(14)
            AHEAD_CASE(15) AHEAD_CASE(16)
#undef AHEAD_CASE
            default: return rocml_fail("gemm: no kernel of that many waves");
        }
    } else {
    constexpr int LDS = 2 * MT * 16 * GS_ROW * 16;
    // Up to 16 rows: four waves per block, or two for the wide products that cannot be split
    // (more, smaller blocks keep more loads in flight when nothing else multiplies their
    // number), about 512 blocks.  Beyond 16 rows the kernel that requests two steps ahead, with
    // eight waves per block (LDS for the activations limits a CU to two blocks at 64 rows;
    // eight waves double the weight bytes in flight per CU and halve the times the activations
    // are read), about 256 blocks.
    constexpr bool AHEAD = MT > 1;
    constexpr int WIDE = AHEAD ? 8 : 4;
    static bool ready = false;
    if (!ready) {
        if constexpr (AHEAD) {
            if (allow_lds(gemm_skinny_ahead_kernel<MT, EPI, false, WIDE>, LDS, "gemm")) return 1;
            if (allow_lds(gemm_skinny_ahead_kernel<MT, EPI, true, WIDE>, LDS, "gemm")) return 1;
        } else {
            if (allow_lds(gemm_skinny_kernel<MT, EPI, false, WIDE>, LDS, "gemm")) return 1;
            if (allow_lds(gemm_skinny_kernel<MT, EPI, true, WIDE>, LDS, "gemm")) return 1;
        }
        ready = true;
    }
    // ("wide" is a product whose blocks of four waves alone are four to a CU or more)
    bool narrow = MT == 1 && n >= 256 * cus;
    int blocks_n = ceil_div(n, narrow ? 32 : 16 * WIDE);
    int target = AHEAD ? cus : 2 * cus;
    int splits = target / blocks_n;
    int by_k = k / 512;
    if (splits > by_k) splits = by_k;
    if (splits > plan.max_splits) splits = plan.max_splits;
    if (splits < 1 || narrow) splits = 1;
    long long per_split = (long long)m * n * sizeof(float);
    if (splits > 1 && (long long)splits * per_split > workspace_bytes)
        splits = workspace ? (int)(workspace_bytes / per_split) : 1;
    if (splits < 1) splits = 1;
    int k_per_split = round_up(ceil_div(k, splits), GS_KC);
    splits = ceil_div(k, k_per_split);
    dim3 grid(blocks_n, splits);
    if (!narrow && workspace) {
        BlockChoice usual{WIDE, splits, k_per_split};
        BlockChoice c = choose_blocks(usual, m, MT, n, k, cus, workspace_bytes, MT == 4 ? 13 : 17, MT == 4 ? 15 : 17, plan.max_splits);
        if (c.splits > 1 && (c.waves != usual.waves || c.splits != usual.splits)) {
            int rc = 1;
            switch (c.waves) {
#define AHEAD_CASE(W_) case W_: rc = launch_ahead_split<MT, W_>(x, ldx, w, ldw, workspace, m, n, k, c.splits, c.k_per_split, stream); break;
                AHEAD_CASE(2) AHEAD_CASE(3) AHEAD_CASE(4) AHEAD_CASE(5) AHEAD_CASE(6) AHEAD_CASE(7) AHEAD_CASE(8)
                AHEAD_CASE(9) AHEAD_CASE(10) AHEAD_CASE(11) AHEAD_CASE(12) AHEAD_CASE(13) AHEAD_CASE(14)
                AHEAD_CASE(15) AHEAD_CASE(16)
#undef AHEAD_CASE
                default: return rocml_fail("gemm: no kernel of that many waves");
            }
            if (rc) return rc;
            if (plan.defer && ldo == n) {
                *plan.deferred = c.splits;
                return 0;
            }
            long long total = (long long)m * n;
            gemm_splitk_reduce_kernel<EPI><<<ceil_div(total, 256), 256, 0, stream>>>(
                (const float*)workspace, out, ldo, m, n, c.splits);
            return 0;
        }
    }
    if (splits == 1 && narrow) {
        if constexpr (MT == 1)
            gemm_skinny_kernel<MT, EPI, false, 2><<<grid, 128, LDS, stream>>>(
                (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, k_per_split);
    } else if (splits == 1) {
        if constexpr (AHEAD)
            gemm_skinny_ahead_kernel<MT, EPI, false, WIDE><<<grid, 64 * WIDE, LDS, stream>>>(
                (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, k_per_split);
        else
            gemm_skinny_kernel<MT, EPI, false, WIDE><<<grid, 64 * WIDE, LDS, stream>>>(
                (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, k_per_split);
    } else {
        if constexpr (AHEAD)
            gemm_skinny_ahead_kernel<MT, EPI, true, WIDE><<<grid, 64 * WIDE, LDS, stream>>>(
                (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, workspace, n, m, n, k, k_per_split);
        else
            gemm_skinny_kernel<MT, EPI, true, WIDE><<<grid, 64 * WIDE, LDS, stream>>>(
                (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, workspace, n, m, n, k, k_per_split);
        if (plan.defer && ldo == n) {
            // the caller's next kernel adds the partial sums itself
            *plan.deferred = splits;
            return 0;
        }
        long long total = (long long)m * n;
        gemm_splitk_reduce_kernel<EPI><<<ceil_div(total, 256), 256, 0, stream>>>(
            (const float*)workspace, out, ldo, m, n, splits);
    }
    return 0;
    }
}

// At most 16 rows: blocks of 16 weight rows, K split over the block's waves and, while there are
// fewer than four blocks a CU, over blocks as well (each wave keeps at least 256 of K).
template <int EPI>
static int launch_kpar(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m, int n, int k,
                       void* workspace, long long workspace_bytes, SplitPlan plan, hipStream_t stream) {
    int n_tiles = ceil_div(n, 16);
    int splits = 4 * cu_count() / n_tiles;
    int by_k = k / 1024;
    if (splits > by_k) splits = by_k;
    if (splits > plan.max_splits) splits = plan.max_splits;
    if (splits < 1 || EPI == EPI_SWIGLU) splits = 1;
    long long per_split = (long long)m * n * sizeof(float);
    if (splits > 1 && (long long)splits * per_split > workspace_bytes)
        splits = workspace ? (int)(workspace_bytes / per_split) : 1;
    if (splits < 1) splits = 1;
    int k_per_split = round_up(ceil_div(k, splits), 128);
    splits = ceil_div(k, k_per_split);
    dim3 grid(n_tiles, splits);
    if (splits == 1) {
        gemm_kpar_kernel<EPI, false><<<grid, GK_THREADS, 0, stream>>>(
            (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, out, ldo, m, n, k, k_per_split, plan.rs);
    } else {
        gemm_kpar_kernel<EPI, true><<<grid, GK_THREADS, 0, stream>>>(
            (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, workspace, n, m, n, k, k_per_split, RowScale{});
        if (plan.defer && ldo == n) {
            *plan.deferred = splits;
            return 0;
        }
        long long total = (long long)m * n;
        gemm_splitk_reduce_kernel<EPI><<<ceil_div(total, 256), 256, 0, stream>>>(
            (const float*)workspace, out, ldo, m, n, splits);
    }
    return 0;
}

template <int EPI>
static int launch_skinny_m(const void* x, int ldx, const void* w, int ldw, void* out, int ldo, int m, int n,
                           int k, void* workspace, long long workspace_bytes, SplitPlan plan, hipStream_t stream) {
    if (m <= 16) return launch_skinny<1, EPI>(x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
    if (m <= 32) return launch_skinny<2, EPI>(x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
    if (m <= 48) return launch_skinny<3, EPI>(x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
    return launch_skinny<4, EPI>(x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
}

// Gated activation over a 32-bit [M, N] product with (gate, up) column pairs: the unfused path of
// the epilogue above, for the kernels that cannot fuse it.
template <typename TO>
__global__ void swiglu_pairs_kernel(const float* __restrict__ gu, TO* __restrict__ out, int ldo, int m, int half) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)m * half) return;
    int r = (int)(idx / half), j = (int)(idx - (long long)r * half);
    const float* row = gu + (size_t)r * 2 * half;
    Elem<TO>::store(out + (size_t)r * ldo + j, silu_mul(row[2 * j], row[2 * j + 1]));
}

// out (+)= sum of split-K partial sums [splits][M][N] in split order: the step that a deferred
// product leaves to its caller, as a kernel of its own.
ROCML_EXPORT int rocml_splitk_reduce(const float* partials, void* out, int out_dtype, int ldo, int m, int n,
                                     int splits, int accumulate, hipStream_t stream) {
    ROCML_REQUIRE(m >= 0 && n > 0 && splits > 0 && ldo >= n, "splitk_reduce: bad sizes M=%d N=%d splits=%d", m, n, splits);
    ROCML_REQUIRE(!accumulate || out_dtype == ROCML_F32, "splitk_reduce: accumulation needs a 32-bit output");
    if (m == 0) return 0;
    int grid = ceil_div((long long)m * n, 256);
    if (accumulate) gemm_splitk_reduce_kernel<EPI_ACC><<<grid, 256, 0, stream>>>(partials, out, ldo, m, n, splits);
    else if (out_dtype == ROCML_F32) gemm_splitk_reduce_kernel<EPI_F32><<<grid, 256, 0, stream>>>(partials, out, ldo, m, n, splits);
    else if (out_dtype == ROCML_BF16) gemm_splitk_reduce_kernel<EPI_BF16><<<grid, 256, 0, stream>>>(partials, out, ldo, m, n, splits);
    else return rocml_fail("splitk_reduce: unknown output type %d", out_dtype);
    ROCML_CHECK_LAUNCH("splitk_reduce");
    return 0;
}

// resid[M, N] += X * W^T for at most 16 rows of bfloat16 operands, whole sums, and the next norm
// prepared: xg[M, N] = bfloat16(resid * gain) and ssq[M][ceil(N / 16)], the sums of squares of
// every 16 columns of a row (see gemm_residual_prescale_kernel).
ROCML_EXPORT int rocml_gemm_residual_prescale(const void* x, int ldx, const void* w, int ldw, float* resid, int ldr,
                                              const float* gain, void* xg, int ldg, float* ssq, int m, int n, int k,
                                              int waves, hipStream_t stream) {
    ROCML_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_residual_prescale: bad sizes M=%d N=%d K=%d", m, n, k);
    ROCML_REQUIRE(m <= 16, "gemm_residual_prescale: at most 16 rows, got %d", m);
    ROCML_REQUIRE(ldx >= k && ldw >= k && ldr >= n && ldg >= n, "gemm_residual_prescale: row strides (%d, %d, %d, %d) too small",
                  ldx, ldw, ldr, ldg);
    ROCML_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0,
                  "gemm_residual_prescale: K and the operands' row strides must be multiples of 8 and the pointers "
                  "16-byte aligned (K=%d ldx=%d ldw=%d)", k, ldx, ldw);
    ROCML_REQUIRE((uintptr_t)resid % 16 == 0 && (uintptr_t)gain % 16 == 0 && (uintptr_t)xg % 8 == 0,
                  "gemm_residual_prescale: the residual stream, the gain and the prepared operand must be aligned");
    ROCML_REQUIRE(resid && gain && xg && ssq, "gemm_residual_prescale: null pointer");
    if (m == 0) return 0;
    int tiles = ceil_div(n, 16);
    ROCML_REQUIRE(waves == 0 || waves == 4 || waves == 8 || waves == 16, "gemm_residual_prescale: 4, 8 or 16 waves, got %d", waves);
    // waves: 0 = choose: eight a block when each still gets 512 of K and the chip holds all blocks
    // of eight at once, else four
    if (waves == 0) waves = (k >= 4096 && tiles <= cu_count()) ? 8 : 4;
#define GRP_LAUNCH(W_)                                                                                          \
    gemm_residual_prescale_kernel<W_><<<tiles, 64 * W_, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, resid, \
                                                                     ldr, gain, (bf16_t*)xg, ldg, ssq, tiles, m, n, k)
    if (waves == 16) GRP_LAUNCH(16);
    else if (waves == 8) GRP_LAUNCH(8);
    else GRP_LAUNCH(4);
#undef GRP_LAUNCH
    ROCML_CHECK_LAUNCH("gemm_residual_prescale");
    return 0;
}

// Whether rocml_gemm_residual_prescale is the faster way to add this product to the residual
// stream and norm the result.  Its blocks own 16 columns and all of K, so the chip must hold them in
// one round, and a CU pulls a block's weight rows at a limited rate, so K must be short or the
// blocks must be nearly one a CU.  Measured in replayed graphs against the product cut along K over
// blocks plus the norm kernel (us): 4096 x 4096 10.3 against 13.8 at 1 row, 12.1 against 14.5 at
// 8, 13.0 against 14.8 at 16; 1024 x 3072 7.6 against 9.2 at 1 row, 9.4 against 9.7 at 16;
// 4096 x 12288 22.8 against 25.6 at 2 rows, 25.3 against 26.6 at 8, 27.9 against 27.3 at 12 (every
// block reads all activations, which is what more rows cost); 2560 x 9728 (160 blocks) 18.4 against
// 17.4 and 5120 x 5120 (320 blocks, more than a round) 19.2 against 17.9 at 1 row: not taken.
ROCML_EXPORT int rocml_gemm_residual_prescale_pays(int m, int n, int k) {
    if (m < 1 || m > 16 || k % 8 != 0) return 0;
    int tiles = ceil_div(n, 16);
    const int cus = cu_count();
    if (tiles > cus) return 0;
    if (k <= 4096) return 1;
    return k <= 12288 && m <= 8 && 10 * tiles >= 9 * cus;
}

// algo: 0 = choose, 1 = plain tiled kernel, 2 = MFMA tile kernel (128x128 tiles), 3 = MFMA few-rows
// kernel (M <= 64), 4 = MFMA kernel for at most 16 rows, 5 to 9 = MFMA tile kernel with 256x256,
// 256x192, 128x192, 256x96 and 64x256 tiles.
// accumulate: out += product (out must be 32-bit); this is the residual sum's epilogue.
// epilogue: 0 = none; 1 = gated activation: W's rows are (gate_j, up_j) pairs and out is
//   [M, N/2] = silu(gate) * up.
// defer: if the product was split along K, leave the partial sums [splits][M][N] at the start of
//   the workspace and report their number in *deferred_splits (0 if the product is complete);
//   the caller's next kernel adds them.  Needs a dense out (ldo == N).
// workspace: device memory for split-K partial sums (may be null: no split).
// row_ssq (may be null): X is bfloat16(x * gain) of a norm over K values whose scale is still to
//   come: row_ssq[M][row_parts] are sums of squares of x whose total over a row gives the row's
//   scale 1 / sqrt(total / K + row_eps), which the gated epilogue applies to its sums.  Only for
//   the gated epilogue of at most 16 rows on the MFMA path.
// max_splits: the most pieces K may be cut into (0: the kernels' own limit of 16), for a caller
//   whose next kernel adds a few partial sums cheaply and more of them one after the other.
ROCML_EXPORT int rocml_gemm(const void* x, int x_dtype, int ldx, const void* w, int w_dtype, int ldw,
                            void* out, int out_dtype, int ldo, int m, int n, int k, int accumulate,
                            int algo, int epilogue, int defer, int* deferred_splits, void* workspace,
                            long long workspace_bytes, const float* row_ssq, int row_parts, float row_eps,
                            int max_splits, hipStream_t stream) {
    if (deferred_splits) *deferred_splits = 0;
    ROCML_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm: bad sizes M=%d N=%d K=%d", m, n, k);
    bool gated = epilogue == 1;
    ROCML_REQUIRE(epilogue == 0 || epilogue == 1, "gemm: unknown epilogue %d", epilogue);
    ROCML_REQUIRE(!gated || (n % 2 == 0 && !accumulate), "gemm: the gated epilogue needs an even N and no accumulation");
    int out_cols = gated ? n / 2 : n;
    ROCML_REQUIRE(ldx >= k && ldw >= k && ldo >= out_cols, "gemm: row strides (%d, %d, %d) below (K, K, N)",
                  ldx, ldw, ldo);
    ROCML_REQUIRE(!accumulate || out_dtype == ROCML_F32, "gemm: accumulation needs a 32-bit output");
    ROCML_REQUIRE(algo >= ALGO_AUTO && algo <= ALGO_MFMA_TILE64X256, "gemm: unknown algorithm %d", algo);
    ROCML_REQUIRE(!defer || deferred_splits, "gemm: deferring needs a place to report the splits");
    if (m == 0) return 0;
    bool bf16_in = x_dtype == ROCML_BF16 && w_dtype == ROCML_BF16;
    bool mfma_ok = bf16_in && k % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 &&
                   ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && (!gated || out_dtype == ROCML_BF16);
    if (algo >= ALGO_MFMA_TILE)
        ROCML_REQUIRE(mfma_ok, "gemm: the MFMA kernels need bfloat16 operands, K and row strides that are "
                               "multiples of 8 and 16-byte aligned pointers (K=%d ldx=%d ldw=%d)", k, ldx, ldw);
    if (algo == ALGO_MFMA_SKINNY)
        ROCML_REQUIRE(m <= 64, "gemm: the few-rows kernel takes at most 64 rows, got %d", m);
    if (algo == ALGO_MFMA_KPAR)
        ROCML_REQUIRE(m <= 16, "gemm: the 16-rows kernel takes at most 16 rows, got %d", m);
    ROCML_REQUIRE(out_dtype == ROCML_F32 || out_dtype == ROCML_BF16, "gemm: unknown output type %d", out_dtype);
    int epi = gated ? EPI_SWIGLU : accumulate ? EPI_ACC : (out_dtype == ROCML_BF16 ? EPI_BF16 : EPI_F32);
    bool use_mfma = mfma_ok && algo != ALGO_PLAIN;
    if (row_ssq)
        ROCML_REQUIRE(gated && m <= 16 && use_mfma && row_parts > 0 && row_eps > 0.f &&
                          (algo == ALGO_AUTO || algo == ALGO_MFMA_SKINNY || algo == ALGO_MFMA_KPAR),
                      "gemm: a row scale goes with the gated epilogue of at most 16 rows on the few-rows MFMA kernels "
                      "(M=%d parts=%d)", m, row_parts);
    if (use_mfma) {
        // Up to 16 rows the few-rows kernels; up to 64 rows still for the gated product (it cannot
        // cut K in pieces, which is what the tile kernel lives on with so few rows) and, up to 48
        // rows, for every product but the widest (the output projection over the vocabulary): with
        // blocks chosen for the busiest CU they are 1 to 7 % ahead of the tile kernel at 48 rows
        // and 4 to 9 % behind it at 64.
        const int cus = cu_count();
        bool few_rows = m <= 16 || (m <= 64 && (gated || (m <= 48 && n < 256 * cus)));
        bool skinny = algo == ALGO_MFMA_SKINNY || (algo == ALGO_AUTO && few_rows);
        SplitPlan plan{defer, deferred_splits, RowScale{row_ssq, row_parts, row_eps, 1.0f / (float)k},
                       max_splits >= 1 && max_splits < 16 ? max_splits : 16};
        int rc;
#define BY_EPI(fn, ...)                                              \
        (epi == EPI_F32 ? fn<EPI_F32>(__VA_ARGS__)                   \
         : epi == EPI_BF16 ? fn<EPI_BF16>(__VA_ARGS__)               \
         : epi == EPI_ACC ? fn<EPI_ACC>(__VA_ARGS__) : fn<EPI_SWIGLU>(__VA_ARGS__))
        // One or two rows (but not the gated product, which has its own choice of blocks): the
        // kernel whose waves split K, unless the output is narrow (fewer than
        // one and a half blocks of 16 weight rows a CU: 4096 or 5120 wide on 256 CUs, the products
        // that return to the hidden size): its blocks are then so few that K must be cut across
        // blocks as well and a wave is left with one chunk; the few-rows kernel is 10 to 15 %
        // faster there.  Beyond two rows the activations
        // read from L2 cost more than the block sharing of the few-rows kernel.
        bool kpar = algo == ALGO_MFMA_KPAR || (algo == ALGO_AUTO && m <= 2 && !gated && 2 * (n / 16) >= 3 * cus);
        if (kpar) rc = BY_EPI(launch_kpar, x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
        else if (skinny) rc = BY_EPI(launch_skinny_m, x, ldx, w, ldw, out, ldo, m, n, k, workspace, workspace_bytes, plan, stream);
        else rc = BY_EPI(launch_mfma_tile, x, ldx, w, ldw, out, ldo, m, n, k,
                         algo == ALGO_MFMA_TILE ? 1 : algo == ALGO_MFMA_TILE256 ? 2 : algo == ALGO_MFMA_TILE192 ? 3
                         : algo == ALGO_MFMA_TILE128X192 ? 4 : algo == ALGO_MFMA_TILE256X96 ? 5
                         : algo == ALGO_MFMA_TILE64X256 ? 6 : 0,
                         workspace, workspace_bytes,
                         plan, stream);
#undef BY_EPI
        if (rc) return rc;
        ROCML_CHECK_LAUNCH("gemm");
        return 0;
    }
    // plain kernel; the gated epilogue runs as a second kernel over a 32-bit product in the workspace
    void* dst = out;
    int dst_ld = ldo, dst_dtype = out_dtype;
    if (gated) {
        ROCML_REQUIRE(workspace && workspace_bytes >= (long long)m * n * (long long)sizeof(float),
                      "gemm: the gated epilogue needs %lld bytes of workspace", (long long)m * n * 4);
        dst = workspace;
        dst_ld = n;
        dst_dtype = ROCML_F32;
    }
    if (x_dtype == ROCML_F32 && w_dtype == ROCML_F32 && dst_dtype == ROCML_F32) {
        launch_gemm_tile<float, float, float>(x, ldx, w, ldw, dst, dst_ld, m, n, k, accumulate, stream);
    } else if (bf16_in && dst_dtype == ROCML_F32) {
        launch_gemm_tile<bf16_t, bf16_t, float>(x, ldx, w, ldw, dst, dst_ld, m, n, k, accumulate, stream);
    } else if (bf16_in && dst_dtype == ROCML_BF16) {
        launch_gemm_tile<bf16_t, bf16_t, bf16_t>(x, ldx, w, ldw, dst, dst_ld, m, n, k, 0, stream);
    } else {
        return rocml_fail("gemm: unsupported type triple x=%d w=%d out=%d", x_dtype, w_dtype, out_dtype);
    }
    if (gated) {
        long long total = (long long)m * (n / 2);
        if (out_dtype == ROCML_F32)
            swiglu_pairs_kernel<float><<<ceil_div(total, 256), 256, 0, stream>>>((const float*)dst, (float*)out, ldo, m, n / 2);
        else
            swiglu_pairs_kernel<bf16_t><<<ceil_div(total, 256), 256, 0, stream>>>((const float*)dst, (bf16_t*)out, ldo, m, n / 2);
    }
    ROCML_CHECK_LAUNCH("gemm");
    return 0;
}
