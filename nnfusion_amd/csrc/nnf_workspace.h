// Scratch-memory sizes of the launcher entry points and the tile plan they follow: pure host
// arithmetic, shared by the library (nnf_*_workspace_bytes, the GEMM dispatcher) and by the emitters,
// which reserve the scratch tensor at compile time.  Nothing here may depend on the device at hand.
#pragma once

#include <math.h>
#include <stddef.h>

namespace nnf
{
    namespace workspace
    {
        inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

        // ---- tile plan of the W8A8 MFMA GEMM (w8a8_gemm_dl.hip) ----------------------------------------
        enum GemmTile
        {
            GEMM_TILE_BIG = 0,   // 256 x 256 outputs
            GEMM_TILE_MID = 1,   // 128 x 128
            GEMM_TILE_SMALL = 2, //  64 x 256
            GEMM_TILE_TINY = 3,  //  32 x 256 (not built for W8A8)
            GEMM_TILE_TALL = 4,  // 256 x 128 (W8A8 only: fills the chip where 256 x 256 tiles leave CUs idle)
        };
        struct GemmPlan
        {
            int tile = GEMM_TILE_BIG;
            int splits = 1; // K ranges; > 1 (and always for the small and tiny tiles): partial sums + a reduction pass
            bool reduce_pass = false;
        };
        constexpr int PLAN_CUS = 256; // the plan is made for the CU count of an MI355X

        inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

        // Estimated run time (seconds) of one tile shape and split count, from rates measured on an MI355X with
        // N(0,1) activations (the GEMMs are power bound: ~950 / 700 / 450 TFLOP/s for the three tile shapes when
        // every CU has a workgroup, and a CU runs faster when fewer are busy: hence the square root), ~6 TB/s for
        // the partial sums (written, then read by the reduction pass) and ~3 us for the second launch.
        // w8a8: the same tiles on the int8 matrix cores (~1870 / 1450 / 900 TOP/s, 1700 for 256 x 128; its weight bytes
        // differ too, but a memory-bound W8A8 shape is decided by the partial-sum term either way)
        inline double estimate_gemm(int M, int N, int K, bool gate, int tile, int splits, bool w8a8)
        {
            const int bm = tile == GEMM_TILE_BIG || tile == GEMM_TILE_TALL ? 256 : tile == GEMM_TILE_MID ? 128 : tile == GEMM_TILE_SMALL ? 64 : 32;
            const int bn = tile == GEMM_TILE_BIG ? (gate ? 128 : 256) : tile == GEMM_TILE_MID || tile == GEMM_TILE_TALL ? 128 : 256;
            static const double rates[2][5] = {{950e12, 700e12, 450e12, 300e12, 800e12}, {1870e12, 1450e12, 900e12, 600e12, 1700e12}};
            const double rate = rates[w8a8 ? 1 : 0][tile];
            const int tiles_m = ceil_div(M, bm), tiles_n = ceil_div(N, bn);
            const double blocks = (double)tiles_m * tiles_n * splits;
            const double rounds = (double)(((long long)blocks + PLAN_CUS - 1) / PLAN_CUS);
            const double util = blocks / (rounds * PLAN_CUS);
            const double n_total = (gate ? 2.0 : 1.0) * N;
            const double flops = 2.0 * tiles_m * bm * n_total * K; // whole tile rows are computed
            double t = flops / (rate * sqrt(util));
            const double weight_time = n_total * K / 2.0 / 4e12;
            if (t < weight_time)
                t = weight_time;
            if (splits > 1 || tile == GEMM_TILE_SMALL || tile == GEMM_TILE_TINY)
                t += 2.0 * splits * M * n_total * 4.0 / 6e12 + 3e-6;
            return t;
        }

        // N: output columns.  forced_tile >= 0 / forced_splits > 0 override the choice (a caller's plan argument).
        inline GemmPlan plan_gemm(int M, int N, int K, bool gate, bool w8a8, int forced_tile, int forced_splits)
        {
            static const int split_options[] = {1, 2, 3, 4, 6, 8, 12, 16};
            const int G = K / 128;
            GemmPlan best;
            double best_t = -1.0;
            for (int tile = GEMM_TILE_BIG; tile <= GEMM_TILE_TALL; ++tile)
            {
                // (forced_tile -2: 256-row tiles, their width left to the plan)
                if (tile == GEMM_TILE_TALL && !w8a8)
                    continue;
                if (forced_tile >= 0 ? tile != forced_tile
                    : forced_tile == -2 ? (tile != GEMM_TILE_BIG && tile != GEMM_TILE_TALL)
                                     : (((tile == GEMM_TILE_BIG || tile == GEMM_TILE_TALL) && M <= 128) ||
                                        (tile == GEMM_TILE_SMALL && M > 64) || (tile == GEMM_TILE_MID && M <= 64) ||
                                        (tile == GEMM_TILE_TINY && (M > 32 || w8a8))))
                    continue;
                for (int s : split_options)
                {
                    // every split keeps at least four groups (eight K steps)
                    if (forced_splits > 0 ? s != 1 : (s > 1 && G / s < 4))
                        continue;
                    const int splits = forced_splits > 0 ? (forced_splits < G ? forced_splits : G) : s;
                    const double t = estimate_gemm(M, N, K, gate, tile, splits, w8a8);
                    if (best_t < 0.0 || t < best_t)
                    {
                        best_t = t;
                        best.tile = tile;
                        best.splits = splits;
                    }
                }
            }
            best.reduce_pass = best.splits > 1 || best.tile == GEMM_TILE_SMALL || best.tile == GEMM_TILE_TINY;
            return best;
        }
        inline GemmPlan plan_w8a8_gemm(int M, int N, int K, int forced_tile = -1, int forced_splits = 0)
        {
            return plan_gemm(M, N, K, false, true, forced_tile, forced_splits);
        }
        // a caller's tile_rows / tile_cols as a forced tile of plan_w8a8_gemm (-1: none; -2: 256-row tiles of the
        // plan's own width)
        inline int w8a8_forced_tile(int tile_rows, int tile_cols)
        {
            if (tile_rows == 256)
                return tile_cols == 256 ? GEMM_TILE_BIG : tile_cols == 128 ? GEMM_TILE_TALL : -2;
            return tile_rows == 128 ? GEMM_TILE_MID : tile_rows == 64 ? GEMM_TILE_SMALL : -1;
        }
        inline size_t gemm_partial_bytes(int M, int N, bool gate, const GemmPlan& p)
        {
            return p.reduce_pass ? align256((size_t)p.splits * M * (gate ? 2 : 1) * N * sizeof(float)) : 0;
        }

        // ---- plan of the fp16 x int4 tile GEMM (w4a16_gemm_sk.h) ----------------------------------------------
        // Tiles of tile_rows x 256 weight rows (SiLU-gate: 128 gate + 128 up rows, i.e. 128 output columns) or, for
        // the products without SiLU-gate, tile_rows x 128; the
        // (tile, superstep of 256 k) units of the whole product are split evenly over `grid` workgroups, one per CU.
        // A tile whose units belong to more than one workgroup is summed through the workspace: slots of
        // tile_rows x 256 fp32; workgroup v parks the first segment of its range in slot v and a later one in slot
        // grid + v; a second launch adds them up.
        struct SkPlan
        {
            int tile_rows = 0; // 32, 64, 128 or 256
            int tile_weight_rows = 256; // weight rows of a tile: 256, or 128 (narrow tiles: plain product only)
            int tiles_m = 0, tiles_n = 0;
            int supersteps = 0; // per tile: ceil(K / 256)
            long long units = 0;
            int grid = 0;
            int slots = 0;     // 0: every tile belongs to one workgroup (no workspace, no second launch)
            size_t bytes() const { return (size_t)slots * tile_rows * tile_weight_rows * sizeof(float); }
            // Synchronisation words for the one-launch form: two for RMSNorm's rstd[] computed inside the launch, then
            // two per tile (workgroups that share a tile add its parts up themselves).  0: no tile is shared and (rms)
            // there is no RMSNorm
            size_t sync_bytes(bool rms = false) const { return (slots || rms) ? ((size_t)tiles_m * tiles_n + 1) * 2 * sizeof(unsigned) : 0; }
        };
        // Tile shape.  What the caller fixes (forced_rows 32 / 64 / 128 / 256, forced_cols 128 / 256) is kept, the rest
        // is chosen by M and N (measured at N = K = 8192 and on the Llama shapes, the candidates in turns in one process):
        // 256 x 256 tiles touch every weight once per 256 rows and are the fastest from about 1500 rows on.  Below, every
        // output tile is shared by several workgroups and what a workgroup parks counts: up to 128 rows 128 x 128 tiles
        // (64 x 128 up to 64); above, 256 x 128 where M fills the 256-row tiles (an even number of 128-row blocks, or
        // less than a seventh of the rows wasted: M = 144 .. 256 40.8 - 42.2 us against 42.8 - 44.3 on 128 x 128 tiles,
        // M = 896 116 against 144) and 128 x 256 where it does not (an odd number of blocks: M = 288 .. 384 61.3 - 62.7
        // against 63.9 - 66.1, M = 576 .. 640 96 against 104); 128 x 128 again where 256-row tiles would leave fewer
        // than 64 tiles (N = 4096 at M = 192 .. 256).  SiLU-gate needs the gate | up halves of a 256-row weight tile;
        // 32-row tiles exist 256 wide only.
        inline void sk_tile_shape(int M, int N, bool gate, int forced_rows, int forced_cols, int& rows, int& cols)
        {
            const bool rows_forced = forced_rows == 32 || forced_rows == 64 || forced_rows == 128 || forced_rows == 256;
            if (rows_forced)
            {
                rows = forced_rows;
                cols = (forced_cols == 128 && !gate && rows != 32) ? 128 : 256;
                return;
            }
            cols = 256;
            if (gate || M <= 32 || M > 1536)
            {
                rows = M <= 32 ? 32 : M <= 64 ? 64 : M <= 1536 ? 128 : 256;
                return;
            }
            if (forced_cols == 256)
            {
                const int padded = ceil_div(M, 256) * 256;
                rows = M <= 64 ? 64 : M <= 128 ? 128 : ((padded - M) * 8 <= M ? 256 : 128);
                return;
            }
            cols = 128;
            rows = M <= 64 ? 64 : 128;
            if (M <= 128)
                return;
            const int blocks = ceil_div(M, 128), padded = ceil_div(M, 256) * 256;
            if ((blocks & 1) == 0 || (padded - M) * 7 <= padded)
            {
                if ((padded / 256) * ceil_div(N, 128) >= 64)
                    rows = 256;
            }
            else if (forced_cols != 128)
                cols = 256;
        }
        // tiles_n column tiles, `per_tile` units of K per tile, at least `min_units` units per workgroup (unless forced);
        // forced_grid: 0 = the plan's own choice
        inline SkPlan plan_sk(int M, int tiles_n, int per_tile, int min_units, int num_cu, int forced_tile_rows, long long forced_grid)
        {
            SkPlan p;
            const int rows = forced_tile_rows;
            p.tile_rows = rows;
            p.tiles_m = ceil_div(M, rows);
            p.tiles_n = tiles_n;
            const int G = per_tile;
            p.supersteps = G;
            p.units = (long long)p.tiles_m * p.tiles_n * G;
            long long grid = p.units / min_units < 1 ? 1 : p.units / min_units;
            if (grid > num_cu)
                grid = num_cu;
            // Whole tiles, one workgroup each, where the tiles fill at least half of the CUs and the CUs left idle cost
            // less than what sharing tiles costs (parts parked and added up, a second start of the pipeline in the
            // middle of the launch: about 30 us, some seven to eleven units of 256 k).  Measured against the even split
            // on 172 tiles of 128 x 256 (gate | up, M = 256, K = 4096) 76 -> 71 us, on 172 of 256 x 128 (M = 256,
            // N = 22016) 65 -> 55, 160 tiles (M = 640, N = 8192, K = 4096) 64 -> 52, 128 (M = 512, K = 2048) 33 -> 26,
            // 192 at K = 8192 111 -> 105; with 86 or 112 tiles (a third, 44 % of the CUs) the even split stays 4-10 %
            // faster.
            const long long tiles = (long long)p.tiles_m * p.tiles_n;
            if (tiles <= num_cu && 2 * tiles >= num_cu && (long long)G * (num_cu - tiles) <= 11ll * num_cu)
                grid = tiles;
            if (forced_grid > 0)
                grid = forced_grid < p.units ? forced_grid : p.units;
            p.grid = (int)grid;
            bool first_used = false, later_used = false;
            for (int v = 0; v < p.grid; ++v)
            {
                const long long u0 = ((long long)v * p.units) / p.grid, u1 = ((long long)(v + 1) * p.units) / p.grid;
                if (u1 <= u0)
                    continue;
                if (u0 % G != 0 || u1 - u0 < G - u0 % G) // the first segment is not a whole tile
                    first_used = true;
                const long long last_tile_begin = ((u1 - 1) / G) * G;
                if (last_tile_begin > u0 && u1 % G != 0) // a later segment that stops short of its tile's end
                    later_used = true;
            }
            p.slots = later_used ? 2 * p.grid : first_used ? p.grid : 0;
            return p;
        }
        // fp16 x int4: units of 256 k (supersteps), a workgroup keeps at least two (eight K steps of 64)
        // forced_tile_rows / forced_cols: 0 = the plan's own choice (sk_tile_shape)
        inline SkPlan plan_w4a16_sk(int M, int N, int K, bool gate, int num_cu, int forced_tile_rows = 0, long long forced_grid = 0,
                                    int forced_cols = 0)
        {
            if (M <= 0 || N <= 0 || K < 128 || num_cu < 1)
                return SkPlan();
            int rows, cols;
            sk_tile_shape(M, N, gate, forced_tile_rows, forced_cols, rows, cols);
            SkPlan p = plan_sk(M, ceil_div(N, (gate || cols == 128) ? 128 : 256), (K / 128 + 1) / 2, 2, num_cu, rows, forced_grid);
            p.tile_weight_rows = cols;
            return p;
        }

        // the plan with a forced tile height (0 = the plan's own) and a forced number of workgroups per tile (0 = the
        // plan's own grid)
        inline SkPlan plan_w4a16_sk_with(int M, int N, int K, bool gate, int num_cu, int tile_rows, int workgroups_per_tile,
                                         int tile_cols = 0)
        {
            if (workgroups_per_tile <= 0)
                return plan_w4a16_sk(M, N, K, gate, num_cu, tile_rows, 0, tile_cols);
            // (at most one workgroup per unit of 256 k: plan_sk limits the grid to the number of units)
            const SkPlan t = plan_w4a16_sk(M, N, K, gate, num_cu, tile_rows, 0, tile_cols);
            return plan_w4a16_sk(M, N, K, gate, num_cu, tile_rows, (long long)t.tiles_m * t.tiles_n * workgroups_per_tile, tile_cols);
        }

        // ---- plan of the skinny (M <= 16) MFMA GEMV kernel ---------------------------------------------
        constexpr size_t LDS_BYTES_PER_CU = 160 * 1024; // gfx950
        struct SkinnyPlan
        {
            int cps = 0, ks = 0, h = 0; // groups per wavefront and pass, wavefronts per workgroup, passes over K
            bool a_regs = false;        // activations kept in registers
            // LDS bytes: staged activations; correction constants + scales; partial sums.  With a_regs the
            // activations are only staged until every wavefront has copied its share, and the partial sums and the
            // output parking area then reuse that space.
            size_t a_bytes = 0, fixed_bytes = 0, red_bytes = 0;
            size_t lds(size_t parking_bytes) const
            {
                const size_t tail = red_bytes + parking_bytes;
                return fixed_bytes + (a_regs ? (a_bytes > tail ? a_bytes : tail) : a_bytes + tail);
            }
        };
        // one workgroup spans all of K: fewest groups per wavefront first (more wavefronts in flight), two
        // passes beyond 16 * 3 groups
        inline SkinnyPlan plan_w4a16_skinny(int M, int K, int forced_cps = 0)
        {
            SkinnyPlan p;
            const int G = K >> 7;
            // (four groups per wavefront in one pass spill registers and measured 30 % slower than three in two passes)
            static const int options[6][2] = {{1, 1}, {2, 1}, {3, 1}, {3, 2}, {4, 2}, {4, 1}};
            for (const auto& o : options)
            {
                const int ks = (G + o[0] * o[1] - 1) / (o[0] * o[1]);
                if (forced_cps != 0 && o[0] != forced_cps)
                    continue;
                if (ks <= 16)
                {
                    p.cps = o[0];
                    p.h = o[1];
                    p.ks = ks;
                    break;
                }
            }
            if (p.cps == 0)
                return p;
            // the A operand fits in registers up to two groups per wavefront (32 VGPRs)
            p.a_regs = p.cps <= 2 && p.h == 1;
            p.a_bytes = ((size_t)G * 16 + 1) * M * 16;
            p.fixed_bytes = (size_t)G * 64 + 2 * (((size_t)16 * G * 2 + 15) & ~(size_t)15);
            p.red_bytes = (size_t)2 * M * 16 * 16 * 4;
            return p;
        }
        // true when one workgroup can hold the activations (M <= 16 rows of K) in LDS
        inline bool w4a16_skinny_fits(int M, int N, int K, int forced_cps = 0)
        {
            if (M < 1 || M > 16 || K < 128 || (K & 127) || N < 16)
                return false;
            // the scale block of a tile (16 rows x K/128 fp16) is fetched in whole, aligned 16-byte pieces
            if (((size_t)N * (K >> 7) * 2) % 16 != 0)
                return false;
            // the kernel addresses weights and scales with 32-bit offsets from their base
            if ((size_t)N * (size_t)(K >> 1) >= ((size_t)1 << 32))
                return false;
            const SkinnyPlan p = plan_w4a16_skinny(M, K, forced_cps);
            // leave room for the output parking area (a few tiles of M x 16 floats)
            return p.cps != 0 && p.cps <= (K >> 7) && p.lds(16 * 1024) <= LDS_BYTES_PER_CU;
        }

        // M <= 16 shapes whose activations do not fit at once are run over ranges of K whose activations do fit:
        // equal ranges (multiples of 1024 columns, at most 4096) when K divides that way, otherwise ranges of a
        // multiple of 1024 and a shorter last one of at least 1024.  Returns the length of the ranges (of all but
        // the last), or 0 when this does not apply.
        inline int w4a16_skinny_split_range(int M, int N, int K)
        {
            if (M < 1 || M > 16 || N < 16 || K < 2048 || (K & 127) || w4a16_skinny_fits(M, N, K))
                return 0;
            if ((size_t)N * (size_t)(K >> 1) >= ((size_t)1 << 32)) // 32-bit offsets over whole rows
                return 0;
            static const int equal[] = {2, 4, 8, 16};
            for (int s : equal)
            {
                const int r = K / s;
                if (K % s == 0 && (r & 1023) == 0 && r <= 4096 && w4a16_skinny_fits(M, N, r))
                    return r;
            }
            static const int lengths[] = {4096, 3072, 2048, 1024};
            for (int r : lengths)
            {
                const int s = (K + r - 1) / r;
                if (w4a16_skinny_fits(M, N, r) && s <= 16 && K - (s - 1) * r >= 1024)
                    return r;
            }
            return 0;
        }
        // the number of those ranges (0: does not apply)
        inline int w4a16_skinny_ksplits(int M, int N, int K)
        {
            const int r = w4a16_skinny_split_range(M, N, K);
            return r ? (K + r - 1) / r : 0;
        }
        inline size_t skinny_split_bytes(int M, int N_total, int K)
        {
            const int s = w4a16_skinny_ksplits(M, N_total, K);
            return s ? align256((size_t)s * M * N_total * sizeof(float)) : 0;
        }

        // ---- the VALU GEMV (w4a16_gemv.hip): up to four activation rows of K staged in LDS ----
        inline bool w4a16_gemv_valu_fits(int M, int K)
        {
            if (M < 1 || M > 16 || K < 32 || (K % 32) != 0)
                return false;
            const int mb = M >= 4 ? 4 : M;
            return (size_t)mb * ((K + 2047) >> 11) * 4 * 64 * 16 <= LDS_BYTES_PER_CU;
        }
        // ---- which kernel variants of the fp16 x int4 product can serve a shape (values of nnf_w4a16_variant) ----
        inline bool w4a16_variant_fits(int M, int N, int K, int variant, int num_cu = PLAN_CUS);

        // ---- one activation row: the row-streaming GEMV (w4a16_gemv_rows.hip) ----
        // Eight wavefronts per workgroup (one workgroup per CU) measured fastest: sixteen pay the per-wavefront
        // parts of the kernel twice as often, four leave the vector units idle between dependent instructions.
        constexpr int ROWS_WAVES = 8;
        inline int rows_grid(int N, int num_cu) { return N < num_cu ? N : num_cu; } // one workgroup per CU
        struct RowsPlan
        {
            int seg = 0;    // wavefront-wide loads (1 KiB of a weight row) per row and wavefront; 0: not applicable
            int kshift = 0; // log2 of the wavefronts that share a row
            int depth = 0;  // rows in flight per wavefront
            // ring + activations (+ zeros) + their constants + the workgroup's scales + parked outputs + row counters (32 bytes) + the wavefronts' sums of squares for RMSNorm (32 bytes)
            // (gate: N outputs from 2 N weight rows; a workgroup holds the scales of its gate rows and of its up rows as
            // two blocks, each rounded up to whole KiB)
            // group_shift: log2 of the group size; zero_points: a zero point per (row, group): 256 bytes more per ring slot
            // and 64 groups, and a second constant per unit of activations
            size_t lds_bytes(int N, int K, int grid, bool gate = false, int group_shift = 7, bool zero_points = false) const
            {
                const size_t rows = (size_t)(N / grid + 1);                       // outputs of a workgroup, at most
                const size_t a_pad = (((size_t)(K >> 3) + 63) & ~(size_t)63) + 4; // 16-byte units of activations
                const size_t halves = gate ? 2 : 1;
                const size_t slot = (size_t)seg * 1024 + (zero_points ? (size_t)((seg + 1) / 2) * 256 : 0);
                return (size_t)ROWS_WAVES * depth * slot + a_pad * 16 + a_pad * 4 * (zero_points ? 2 : 1) +
                       halves * ((rows * (size_t)(K >> group_shift) * 2 + 1023) & ~(size_t)1023) +
                       ((halves * rows) << kshift) * sizeof(float) + 64;
            }
        };
        // N: outputs (gate: from 2 N weight rows).  forced_depth: 0 = the plan's own choice
        inline RowsPlan plan_w4a16_rows(int M, int N, int K, int num_cu, int forced_depth = 0, bool gate = false,
                                        int group_shift = 7, bool zero_points = false, int bits = 4)
        {
            RowsPlan p;
            // whole 16-byte pieces of scales per segment, 4-byte aligned: K a multiple of 256
            // (the activations are fetched as at most 2048 16-byte units: K <= 16384)
            if (M != 1 || N < 1 || K < 1024 || K > 16384 || (K & 255) || num_cu < 1 || group_shift < 5 || group_shift > 7 ||
                (gate && (group_shift != 7 || zero_points)) || (bits != 4 && (bits != 8 || gate)))
                return p;
            const int loads_per_row = ((bits == 8 ? K : K >> 1) + 1023) >> 10;
            int kshift = 0;
            while ((1 << kshift) <= ROWS_WAVES && (loads_per_row + (1 << kshift) - 1) >> kshift > 3)
                ++kshift;
            if ((1 << kshift) > ROWS_WAVES)
                return p;
            p.kshift = kshift;
            p.seg = (loads_per_row + (1 << kshift) - 1) >> kshift;
            const int grid = rows_grid(N, num_cu);
            // rows per wavefront of a K segment: the first `depth` of them are fixed
            const int rows_q = ((gate ? 2 : 1) * (N / grid)) / (ROWS_WAVES >> kshift);
            // Two rows in flight per wavefront (a CU takes about 64 wavefront-wide loads in flight; more and the
            // wavefronts stall at issue), a little deeper when a wavefront has many rows to walk (measured).
            const int depth_max = p.seg == 3 ? 2 : 4;
            p.depth = forced_depth > 0 ? forced_depth : (rows_q >= 16 ? (p.seg == 1 ? 4 : 3) : 2);
            if (p.depth > depth_max)
                p.depth = depth_max;
            if (p.depth > rows_q)
                p.depth = rows_q < 1 ? 1 : rows_q;
            while (p.depth > 1 && p.lds_bytes(N, K, grid, gate, group_shift, zero_points) > LDS_BYTES_PER_CU)
                --p.depth;
            if (p.lds_bytes(N, K, grid, gate, group_shift, zero_points) > LDS_BYTES_PER_CU)
                p.seg = 0;
            return p;
        }

        // ---- W8A8 ---------------------------------------------------------------------------------------
        constexpr int Q8_SKINNY_CPS = 2; // preferred chunks per wavefront and pass (more in flight measured slower)
        struct Q8SkinnyPlan
        {
            int cps = 0, kh = 0, ks = 0; // 64-byte chunks of K per wavefront and pass, passes, wavefronts
            size_t lds = 0;              // LDS bytes without the output parking area
        };
        inline Q8SkinnyPlan plan_w8a8_skinny(int M, int K, int forced_cps = 0)
        {
            Q8SkinnyPlan pl;
            const int C = K >> 6;
            // chunks per wavefront and tile: the smallest power of two that needs at most 16 wavefronts
            int per_wave = 1;
            while (per_wave <= 16 && (C + per_wave - 1) / per_wave > 16)
                per_wave *= 2;
            if (per_wave > 16)
                return pl;
            int cps = forced_cps > 0 ? forced_cps : Q8_SKINNY_CPS;
            if (cps > per_wave)
                cps = per_wave;
            while (per_wave / cps > 8)
                cps *= 2;
            pl.cps = cps;
            pl.kh = per_wave / cps;
            pl.ks = (C + per_wave - 1) / per_wave;
            pl.lds = (size_t)pl.ks * per_wave * 4 * M * 16 + (size_t)2 * pl.ks * 256 * 4;
            return pl;
        }
        inline bool w8a8_skinny_fits(int M, int K)
        {
            if (M < 1 || M > 16 || (K & 63))
                return false;
            const Q8SkinnyPlan pl = plan_w8a8_skinny(M, K);
            return pl.cps != 0 && pl.lds + 16 * 1024 <= LDS_BYTES_PER_CU;
        }
        // ---- W8A8, 2 .. 32 activation rows: the row-streaming MFMA kernel (w8a8_mrows.hip) ----
        // K a multiple of 256 up to 16384 (12288 for 17 .. 32 rows).
        // One workgroup per CU, eight wavefronts that each own an eighth of K (256 bytes of every 2 KiB) and keep
        // their share of the activations in registers.  LDS: per wavefront a ring of 4-KiB slots, two sets of eight
        // partial tiles (one or two blocks of 16 rows), the workgroup's finished tiles parked until the end.
        // Two slots (64 KiB in flight per CU) measured 2-9 % faster than three.
        constexpr int W8A8_MROWS_SLOTS = 2;
        inline size_t w8a8_mrows_lds_bytes(int M, int slots, int tiles)
        {
            // ring; partial tiles and parked sums -- or, while the kernel starts, two blocks of 16 rows x 256 bytes of
            // activations per wavefront
            const size_t tail = (size_t)2 * 8 * (M <= 16 ? 1 : 2) * 1024 + (size_t)tiles * M * 64;
            const size_t staging = M > 16 ? (size_t)8 * 2 * 4096 : 0;
            return (size_t)8 * slots * 4096 + (tail > staging ? tail : staging);
        }
        inline bool w8a8_mrows_fits(int M, int N, int K, int num_cu)
        {
            if (M < 2 || M > 32 || N < 16 || num_cu < 1)
                return false;
            // ceil(K / 2048) steps per tile (a template parameter): 16 VGPRs of activations per step and block of rows
            if (K < 1024 || K > (M <= 16 ? 16384 : 12288) || (K & 255))
                return false;
            const int n_tiles = (N + 15) / 16;
            const int grid = n_tiles < num_cu ? n_tiles : num_cu;
            return w8a8_mrows_lds_bytes(M, W8A8_MROWS_SLOTS, (n_tiles + grid - 1) / grid) <= LDS_BYTES_PER_CU;
        }
        // Where the library picks it by itself.  Measured alternately on cold weights against the split-K M <= 16 kernel
        // it is level to 10 % faster up to M = 14 (6 % slower at M = 2, N = K = 8192: not taken below eight rows there),
        // 5-30 % faster at M = 16, and 4-38 % faster than the MFMA tile GEMM at M = 17 .. 32.
        // (Where K does not fill the last step, wavefronts fetch bytes that do not count: at least three quarters of what
        // is fetched must count.)
        inline bool w8a8_mrows_preferred(int M, int N, int K, int num_cu)
        {
            if (((K + 2047) >> 11) == 4 && M < 8) // N = K = 8192: 16.2 us at M = 2 against 15.3 (level from M = 8 on)
                return false;
            return w8a8_mrows_fits(M, N, K, num_cu) && 4 * K >= 3 * 2048 * ((K + 2047) >> 11);
        }
        // Two ranges of K, added up inside the launch (given synchronisation words: one per workgroup of a range, and room for
        // the int32 sums of the ranges): every workgroup fetches all M x K activations ahead of its first MFMA, over two ranges
        // half of them.  Measured (8 .. 32 rows, N = 4096 .. 8192, K = 8192 and 14336) 0.8 - 1.3 us faster than one pass;
        // slower at K = 4096, with more than four tiles per workgroup (N = 16384: +3 us) and over four ranges.
        inline int w8a8_mrows_ranges(int M, int N, int K, int num_cu)
        {
            const int per_range = num_cu / 2;
            if (M < 8 || K < 8192 || (K & 511) || per_range < 1 || (N + 15) / 16 > 4 * per_range)
                return 1;
            // (17 .. 32 rows, whose activations arrive as whole lines: only where a workgroup has more than one tile
            // anyway -- N = 4096 at 32 rows: 12.3 us in one pass, 13.0 over two ranges; N = 8192: 20.9 / 19.6)
            if (M > 16 && (N + 15) / 16 <= num_cu)
                return 1;
            return w8a8_mrows_fits(M, N, K / 2, per_range) ? 2 : 1;
        }
        inline size_t w8a8_mrows_ranges_bytes(int M, int N, int K, int num_cu)
        {
            const int ranges = w8a8_mrows_ranges(M, N, K, num_cu);
            return ranges > 1 ? align256((size_t)ranges * M * N * sizeof(int)) : 0;
        }
        // ---- 2 .. 16 activation rows (.. 32 up to K = 4096): the row-streaming MFMA kernel (w4a16_mrows.hip) ----
        // One workgroup per CU, eight wavefronts that each own an eighth of K (GW groups of every step of a tile) and
        // keep their share of the activations in registers.  LDS: per wavefront two slots of GW KiB of weights and of
        // their scales, two sets of eight partial tiles (one or two blocks of 16 rows), and the workgroup's finished
        // tiles parked until the end.
        // Two forms.  K / 1024 = 1, 2, 3, 4, 6, 8: K is a compile-time constant of the kernel.  Any other multiple of
        // 256 up to 8192 (M <= 16): K is a run-time value, two steps of 8 * GW groups with the smallest GW (2, 3, 4)
        // that covers K; wavefronts past the end of K fetch groups that another one already covers and discard them.
        inline bool w4a16_mrows_fixed_k(int M, int K)
        {
            const int kw = K >> 10;
            return !(K & 1023) && kw >= 1 && kw <= 8 && kw != 5 && kw != 7 && (M <= 16 || kw <= 4);
        }
        inline int w4a16_mrows_step_groups(int M, int K) // GW
        {
            const int kw = K >> 10, G = K >> 7;
            if (w4a16_mrows_fixed_k(M, K))
                return (kw & 1) ? kw : kw / 2; // even K / 1024: two steps per tile
            return G <= 32 ? 2 : G <= 48 ? 3 : 4;
        }
        // Whether the kernel brings its activations in through LDS as whole lines or straight into the registers.  Straight
        // in, a load touches two lines of every row for 32 bytes each, four times over; through LDS every line is touched
        // once, but the blocks come one behind the other (0.3 - 0.5 us).  Measured, K = 4096: 2 / 4 / 6 rows 4.84 / 5.07 /
        // 5.20 us straight against 5.19 / 5.27 / 5.29, 8 / 12 / 16 rows 5.63 / 6.52 / 7.3 against 5.30 / 5.40 / 5.55;
        // K = 8192: 4 / 6 rows 12.05 / 12.45 against 11.58 / 11.70; 32 rows at N = K = 4096: 10.8 against 7.1.
        constexpr bool mrows_stages_activations(int M, int K) { return (long long)M * K >= 32768; }
        // the room for that: two blocks of 16 rows x 256 bytes per wavefront, where the partial tiles and parked sums go later
        constexpr size_t mrows_tail_bytes(size_t tail) { return tail > (size_t)8 * 2 * 4096 ? tail : (size_t)8 * 2 * 4096; }
        inline size_t w4a16_mrows_lds_bytes_gw(int gw, int M, int tiles)
        {
            const size_t mb = M <= 16 ? 1 : M <= 32 ? 2 : 4; // blocks of 16 rows
            // ring, scales; partial tiles, the wavefronts' sums of squares per row (RMSNorm inside the kernel), parked sums --
            // or, while the kernel starts, two blocks of 16 rows x 256 bytes of activations per wavefront
            const size_t tail = (size_t)2 * 8 * mb * 1024 + 8 * mb * 64 + (size_t)tiles * M * 64;
            const size_t staging = (size_t)8 * 2 * 4096;
            return (size_t)8 * 2 * gw * 1024 + 8 * 512 + (tail > staging ? tail : staging);
        }
        inline size_t w4a16_mrows_lds_bytes(int K, int M, int tiles)
        {
            return w4a16_mrows_lds_bytes_gw(w4a16_mrows_step_groups(M, K), M, tiles);
        }
        // N: output columns; gate: from 2 N weight rows (a workgroup walks the gate and the up tile of each output tile)
        inline bool w4a16_mrows_fits(int M, int N, int K, int num_cu, bool gate = false)
        {
            if (M < 2 || M > 32 || N < 16 || num_cu < 1 || K < 1024 || K > 8192 || (K & 255))
                return false;
            if (!w4a16_mrows_fixed_k(M, K) && M > 16 && K > 4096) // two blocks of rows: at most four groups per wavefront
                return false;
            const int n_tiles = (N + 15) / 16;
            const int grid = n_tiles < num_cu ? n_tiles : num_cu;
            return w4a16_mrows_lds_bytes(K, M, (gate ? 2 : 1) * ((n_tiles + grid - 1) / grid)) <= LDS_BYTES_PER_CU;
        }
        // The same kernel for groups of 32 / 64 / 128 and zero points per (row, group) (w4a16_mrows_q_kernel): 2 .. 16 rows
        // (.. 32 up to K = 4096), K = 2048, 4096, 8192 (GW = K / 2048 groups of 128 per wavefront and step); per wavefront and ring slot 256 bytes
        // per 64 4-byte words of scales (GW x 128 / group scales for each of 16 rows) and as much again for zero points.
        inline size_t w4a16_mrows_q_lds_bytes(int K, int M, int tiles, int group_shift, bool zero_points)
        {
            const int gw = K >> 11;
            const int words = (gw << (7 - group_shift)) / 2; // of scales per row, step and wavefront
            const int loads = (16 * words + 63) / 64;
            const size_t aux = (size_t)(zero_points ? 2 : 1) * loads * 256;
            const size_t mb = M <= 16 ? 1 : 2; // blocks of 16 rows
            return (size_t)8 * 2 * gw * 1024 + 8 * 2 * aux + mrows_tail_bytes((size_t)2 * 8 * mb * 1024 + (size_t)tiles * M * 64);
        }
        // (17 .. 32 rows: two blocks of rows in registers, up to K = 4096)
        inline bool w4a16_mrows_q_fits(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
        {
            if (M < 2 || M > 32 || (M > 16 && K > 4096) || N < 16 || num_cu < 1 || (K != 2048 && K != 4096 && K != 8192) ||
                group_shift < 5 || group_shift > 7)
                return false;
            if (((K >> 11) << (7 - group_shift)) & 1) // K = 2048 with groups of 128: half a word of scales per step
                return false;
            const int n_tiles = (N + 15) / 16;
            const int grid = n_tiles < num_cu ? n_tiles : num_cu;
            return w4a16_mrows_q_lds_bytes(K, M, (n_tiles + grid - 1) / grid, group_shift, zero_points) <= LDS_BYTES_PER_CU;
        }
        // 8-bit weights, 2 .. 16 rows, up to 32 at K <= 4096 (w8a16_mrows_q_kernel): K = 4096 / 8192 (four 64-byte pieces of a weight row per
        // wavefront and step, two / four steps), K = 2048 with groups of 32 / 64 (two pieces, two steps)
        inline size_t w8a16_mrows_q_lds_bytes(int K, int M, int tiles, int group_shift, bool zero_points)
        {
            const int gw = K == 2048 ? 2 : 4;
            const int spr = (gw * 64) >> group_shift; // scales per row, step and wavefront
            const int loads = (16 * (spr / 2) + 63) / 64 + (zero_points ? (16 * spr + 63) / 64 : 0);
            const size_t mb = M <= 16 ? 1 : 2; // blocks of 16 rows
            return (size_t)8 * 2 * gw * 1024 + (size_t)8 * 2 * loads * 256 + mrows_tail_bytes((size_t)2 * 8 * mb * 1024 + (size_t)tiles * M * 64);
        }
        // (17 .. 32 rows: two blocks of rows in registers, up to K = 4096)
        inline bool w8a16_mrows_q_fits(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
        {
            if (M < 2 || M > 32 || (M > 16 && K > 4096) || N < 16 || num_cu < 1 || (K != 2048 && K != 4096 && K != 8192) || group_shift < 5 ||
                group_shift > 7 || (K == 2048 && group_shift == 7))
                return false;
            const int n_tiles = (N + 15) / 16;
            const int grid = n_tiles < num_cu ? n_tiles : num_cu;
            return w8a16_mrows_q_lds_bytes(K, M, (n_tiles + grid - 1) / grid, group_shift, zero_points) <= LDS_BYTES_PER_CU;
        }
        // ... and with K as a run-time value (w4a16_mrows_q_any_kernel): 2 .. 16 rows, any other multiple of 256.  Up to
        // K = 8192 in one piece (two steps of 8 x gw blocks of 128 weights, when at least three quarters of what the
        // wavefronts fetch counts), above over ranges of at most 32 blocks with fp32 sums per range and the reduction pass
        // (as w4a16_mrows_split does it for groups of 128 with a scalar zero point).
        struct MrowsQAny
        {
            int ranges = 0, range_blocks = 0, gw = 0; // ranges 0: not applicable; 1: no workspace
        };
        inline size_t w4a16_mrows_q_any_lds_bytes(int gw, int M, int tiles, int group_shift, bool zero_points)
        {
            const int spc = 1 << (7 - group_shift);
            const int words = spc == 1 ? gw / 2 + 1 : gw * spc / 2;
            const int loads = (16 * words + 63) / 64;
            const size_t aux = (size_t)(zero_points ? 2 : 1) * loads * 256;
            return (size_t)8 * 2 * gw * 1024 + 8 * 2 * aux + mrows_tail_bytes((size_t)2 * 8 * 1024 + (size_t)tiles * M * 64);
        }
        inline MrowsQAny w4a16_mrows_q_any_plan(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
        {
            MrowsQAny p;
            if (M < 2 || M > 16 || N < 16 || K < 1024 || K > 65536 || (K & 255) || num_cu < 16 || group_shift < 5 || group_shift > 7)
                return p;
            const int B = K >> 7;
            int ranges = 1, rb = B, gw;
            if (K <= 8192)
            {
                gw = B <= 32 ? 2 : B <= 48 ? 3 : 4;
                if (4 * B < 3 * 16 * gw)
                    return p;
            }
            else
            {
                ranges = (B + 31) / 32;
                rb = (((B + ranges - 1) / ranges) + 1) & ~1;
                gw = 2;
                if (B - (ranges - 1) * rb < gw)
                    return p;
            }
            const int n_tiles = (N + 15) / 16, per_range = num_cu / ranges;
            const int grid = n_tiles < per_range ? n_tiles : per_range;
            if (w4a16_mrows_q_any_lds_bytes(gw, M, (n_tiles + grid - 1) / grid, group_shift, zero_points) > LDS_BYTES_PER_CU)
                return p;
            p.ranges = ranges;
            p.range_blocks = rb;
            p.gw = gw;
            return p;
        }
        // The tile GEMM with other block parameters (groups of 32 / 64 / 128, zero points per (row, group)): above 16 rows,
        // K a multiple of 256 (the kernel addresses its operands with 32-bit byte offsets); the plain product, same plan
        inline bool w4a16_gemm_q_fits(int M, int N, int K, int group_shift)
        {
            return M > 16 && N >= 1 && K >= 256 && !(K & 255) && group_shift >= 5 && group_shift <= 7 &&
                   (size_t)M * K * 2 + 8192 < ((size_t)1 << 32) && (size_t)N * (K >> 1) < ((size_t)1 << 32);
        }
        // nnf_wna16_gemm with parameters other than 4 bits / groups of 128 / scalar zero point, 4-bit weights: [ parked tiles ]
        // on the tile GEMM, [ fp32 sums per range of K ] for 2 .. 16 rows with K above 8192; nothing otherwise
        inline size_t wna16_gemm(int M, int N, int K, int bits, int group, int num_cu = PLAN_CUS)
        {
            const int gs = group == 32 ? 5 : group == 64 ? 6 : group == 128 ? 7 : 0;
            if (bits != 4 || gs == 0)
                return 0;
            if (w4a16_mrows_q_fits(M, N, K, gs, true, num_cu)) // up to 32 rows: the row-streaming kernel
                return 0;
            const MrowsQAny any = w4a16_mrows_q_any_plan(M, N, K, gs, true, num_cu); // ... over ranges of K: their fp32 sums
            if (any.ranges > 0)
                return any.ranges > 1 ? align256((size_t)any.ranges * M * N * sizeof(float)) : 0;
            if (!w4a16_gemm_q_fits(M, N, K, gs))
                return 0;
            return plan_w4a16_sk(M, N, K, false, num_cu).bytes();
        }
        // ---- the fused product / MLP block for block parameters that run the nodes one after the other ----------------------
        inline size_t w4a16_gemm(int M, int N, int K, int, int num_cu = PLAN_CUS);
        // nnf_wna16_gemm's own scratch memory, whichever form the zero point takes
        inline size_t wna16_gemm_any(int M, int N, int K, int bits, int group, int num_cu = PLAN_CUS)
        {
            size_t a = wna16_gemm(M, N, K, bits, group, num_cu);
            if (bits == 4 && group == 128)
            {
                const size_t b = w4a16_gemm(M, N, K, group, num_cu);
                a = b > a ? b : a;
            }
            return align256(a);
        }
        // nnf_wna16_gemm_fused: [ RMSNorm(A): M x K fp16 ][ the product, where the epilogue cannot read it from Y: M x rows fp16 ]
        //                       [ the product's own ]
        struct QFusedLayout
        {
            size_t xn = 0, product = 0, gemm = 0;
            size_t total() const { return xn + product + gemm; }
        };
        inline QFusedLayout wna16_fused_layout(int M, int N, int K, int bits, int group, bool rms, bool gate, bool through_scratch)
        {
            QFusedLayout l;
            const int rows = gate ? 2 * N : N;
            l.xn = rms ? align256((size_t)M * K * 2) : 0;
            l.product = (gate || through_scratch) ? align256((size_t)M * rows * 2) : 0;
            l.gemm = wna16_gemm_any(M, rows, K, bits, group);
            return l;
        }
        // nnf_fused_mlp_wna16: [ RMSNorm(x): M x H fp16 ][ gate | up products M x 2I fp16, then the down product M x H fp16 ]
        //                      [ h: M x I fp16 ][ the products' own ]
        inline size_t fused_mlp_wna16(int M, int H, int I, int bits, int group)
        {
            const size_t a = wna16_gemm_any(M, 2 * I, H, bits, group), b = wna16_gemm_any(M, H, I, bits, group);
            const size_t wide = (size_t)(2 * I > H ? 2 * I : H);
            return align256((size_t)M * H * 2) + align256((size_t)M * wide * 2) + align256((size_t)M * I * 2) + (a > b ? a : b);
        }

        // K above 8192 (above 4096 for 17 .. 32 rows, above 2048 for 33 .. 64; a multiple of 256): the run-time-K form over equal ranges of K (in whole pairs of
        // groups; the last range may be shorter), each on its share of the CUs; fp32 sums per range, added by the
        // reduction pass.  Every workgroup fetches the activations of its range, so shorter ranges mean less of that
        // traffic (CUs x M x K / ranges x 2 bytes): ranges of at most 32 groups (GW = 2) measured fastest (K = 11008:
        // 3 ranges, 14336: 4, 28672: 7-8; 10-25 % faster than the fewest ranges that fit the registers).
        struct MrowsSplit
        {
            int ranges = 0, range_groups = 0, gw = 0;
        };
        inline MrowsSplit w4a16_mrows_split(int M, int N, int K, int num_cu)
        {
            MrowsSplit sp;
            // (33 .. 64 rows run on the kernel, but against the tile GEMM, measured alternately: 33 / 40 rows take 25.9 / 27.4 us
            // against 29.1 / 29.3 at N = 22016, K = 4096 and 12.2 / 12.9 against 14.8 / 15.3 at N = K = 4096, are level at K = 8192 and
            // 11008, 8-10 % slower at K = 5120, and slower everywhere from about 48 rows on: taken up to 40 rows and K = 4096)
            // (8 .. 16 rows at K = 8192, up to 8192 weight rows: in one launch every workgroup fetches all M x 8192 activations
            // ahead of its first MFMA; over two ranges it fetches half of them.  With the activations fetched as whole lines
            // that is worth 5 % at 8 rows and nothing at 12 .. 16 (it was 10-18 % before); at 16384 weight rows one range is
            // 6 % faster, and it was slower at K = 5120 / 6144)
            const int longest_single = M <= 16 ? ((M >= 8 && K == 8192 && N <= 8192) ? 8191 : 8192) : M <= 32 ? 4096 : 2048;
            if (M < 2 || M > 40 || N < 16 || K <= longest_single || K > (M <= 32 ? 65536 : 4096) || (K & 255) || num_cu < 16)
                return sp;
            const int G = K >> 7;
            // 33 .. 64 rows: four blocks of rows leave registers for two groups per wavefront: ranges of 16 groups
            int ranges = M <= 32 ? (G + 31) / 32 : (G + 15) / 16;
            const int rg = (((G + ranges - 1) / ranges) + 1) & ~1;
            const int gw = rg <= 16 ? (M <= 32 ? 2 : 1) : rg <= 32 ? 2 : rg <= 48 ? 3 : 4;
            if ((M > 32 && gw > 1) || (M > 16 && gw > 2)) // (only with a forced number of ranges)
                return sp;
            if (G - (ranges - 1) * rg < gw) // the last range holds at least one wavefront's groups
                return sp;
            const int n_tiles = (N + 15) / 16, per_range = num_cu / ranges;
            const int grid = n_tiles < per_range ? n_tiles : per_range;
            if (w4a16_mrows_lds_bytes_gw(gw, M, (n_tiles + grid - 1) / grid) > LDS_BYTES_PER_CU)
                return sp;
            sp.ranges = ranges;
            sp.range_groups = rg;
            sp.gw = gw;
            return sp;
        }
        // synchronisation words for adding the ranges up inside the launch: one per workgroup of a range
        inline size_t mrows_split_sync_bytes(int num_cu) { return (size_t)num_cu * sizeof(unsigned); }
        // Adding the ranges up inside the launch pays while a workgroup has few output tiles: the last arriver adds its
        // tiles up one after the other, the reduction pass works on all of them at once (N = 28672 at 16 rows: 32 us
        // against 30.7 with the pass; N <= 14336: level or up to 8 % faster in the launch).
        inline bool mrows_split_adds_in_launch(int N, int ranges, int num_cu)
        {
            const int per_range = num_cu / ranges > 0 ? num_cu / ranges : 1;
            return ((N + 15) / 16 + per_range - 1) / per_range <= 8;
        }
        inline size_t mrows_split_bytes(int M, int N_total, int K)
        {
            const int r = w4a16_mrows_split(M, N_total, K, PLAN_CUS).ranges;
            return r ? align256((size_t)r * M * N_total * sizeof(float)) : 0;
        }
        // Where the library picks it by itself, from measurements against the split-K MFMA GEMV on cold weights
        // (M = 2 / 16): K = 2048, 4096, 6144, 8192: 0-15 % / 15-30 % faster;  K = 1024, 3072: 5-35 % faster;
        // run-time K: 0-5 % / 15-35 % faster at K = 3584, 5120, 7168 (but up to 19 % slower below eight rows at K = 7168), level
        // at K = 2560, slower at K = 1536 and 2304, where most of what the wavefronts fetch is discarded: taken when at
        // least three quarters of the fetched groups count.
        inline bool w4a16_mrows_preferred(int M, int N, int K, int num_cu, bool gate = false)
        {
            if (!w4a16_mrows_fits(M, N, K, num_cu, gate))
                return false;
            if (w4a16_mrows_fixed_k(M, K))
                return true;
            const int gw = w4a16_mrows_step_groups(M, K);
            if (gw == 4 && M < 8) // K = 6400 .. 7936: N = K = 7168 takes 10.7 us at M = 2 against 9.0 (level from M = 6 on)
                return false;
            return 4 * (K >> 7) >= 3 * 16 * gw;
        }
        // ---- W8A8, one activation row: the row-streaming GEMV (w8a8_gemv_rows.hip) ----
        struct Q8RowsPlan
        {
            int seg = 0;    // wavefront-wide loads (1 KiB of a weight row) per row and wavefront; 0: not applicable
            int kshift = 0; // log2 of the wavefronts that share a row
            int depth = 0;  // rows in flight per wavefront
            // ring + activations (+ zeros) + parked sums + row counters
            size_t lds_bytes(int N, int K, int grid) const
            {
                const size_t rows = (size_t)(N / grid + 1); // of a workgroup, at most
                return (size_t)ROWS_WAVES * depth * seg * 1024 + (((size_t)K + 1023) & ~(size_t)1023) + 16 +
                       (rows << kshift) * sizeof(int) + 64;
            }
        };
        // forced_depth: for experiments (0: the plan's own choice)
        inline Q8RowsPlan plan_w8a8_rows(int M, int N, int K, int num_cu, int forced_depth = 0)
        {
            Q8RowsPlan p;
            if (M != 1 || N < 1 || K < 1024 || (K & 127) || num_cu < 1)
                return p;
            const int loads_per_row = (K + 1023) >> 10;
            int kshift = 0;
            while ((1 << kshift) <= ROWS_WAVES && (loads_per_row + (1 << kshift) - 1) >> kshift > 3)
                ++kshift;
            if ((1 << kshift) > ROWS_WAVES)
                return p; // K > 24576
            p.kshift = kshift;
            p.seg = (loads_per_row + (1 << kshift) - 1) >> kshift;
            const int grid = rows_grid(N, num_cu);
            const int rows_q = (N / grid) / (ROWS_WAVES >> kshift); // rows per wavefront of a K segment
            const int depth_max = p.seg == 3 ? 2 : 4;
            p.depth = forced_depth > 0 ? forced_depth : (rows_q >= 16 ? (p.seg == 1 ? 4 : 3) : 2);
            if (p.depth > depth_max)
                p.depth = depth_max;
            if (p.depth > rows_q)
                p.depth = rows_q < 1 ? 1 : rows_q;
            while (p.depth > 1 && p.lds_bytes(N, K, grid) > LDS_BYTES_PER_CU)
                --p.depth;
            if (p.lds_bytes(N, K, grid) > LDS_BYTES_PER_CU)
                p.seg = 0;
            return p;
        }
        // nnf_w8a8_gemm / nnf_w8a8_gemm_acc: [ int32 partial sums ] (same tile plan as the fp16 x int4 GEMM)
        inline size_t w8a8_gemm(int M, int N, int K)
        {
            if (M <= 0 || N <= 0 || K < 128)
                return 0;
            // (the row-streaming kernel over two ranges of K: the ranges' int32 sums)
            const size_t ranges = w8a8_mrows_preferred(M, N, K, PLAN_CUS) ? w8a8_mrows_ranges_bytes(M, N, K, PLAN_CUS) : 0;
            if (w8a8_skinny_fits(M, K))
                return ranges;
            const size_t tiles = gemm_partial_bytes(M, N, false, plan_w8a8_gemm(M, N, K));
            return tiles > ranges ? tiles : ranges;
        }
        // ---- which kernel serves an fp16 x int4 product, and the scratch memory that launch uses --------------------
        // Decided from the shape, the fused parts asked for and the device's CU count alone: the launcher, the entry
        // points' workspace checks and the *_workspace_bytes queries (for PLAN_CUS) all ask this one function.
        struct W4A16Route
        {
            // NONE: the kernel family asked for cannot serve the shape
            enum Kind { NONE, ROWS, MROWS, SKINNY, MROWS_SPLIT, SKINNY_SPLIT, TILE } kind = NONE;
            int ksplits = 0;          // *_SPLIT: ranges of K (fp32 partial sums, then the reduction pass)
            bool via_scratch = false; // SKINNY: products to scratch first, an element-wise epilogue kernel reads them
            SkPlan plan;              // TILE
            size_t partial_bytes = 0; // partial sums / parked tiles / the products ahead of an element-wise epilogue
            size_t rms_bytes = 0;     // RMSNorm prologue: rstd, fp32 [M] (the kernels multiply the RMSNorm weight in
                                      // themselves), or for the MFMA GEMV kernel the normalised activations, fp16 [M, K]
        };
        // N: output columns (gate: from 2 N weight rows); rms: with the RMSNorm prologue; in_place_residual: the residual
        // is the output buffer itself.  path: 0 the library's order of preference, 2 / 4 one family of GEMV kernels only
        // (values of nnf_w4a16_variant), 3 the tile GEMM with tile_rows / k_parts (0: its own plan).
        inline W4A16Route route_w4a16(int M, int N, int K, bool gate, bool rms, bool in_place_residual, int num_cu, int path = 0,
                                      int tile_rows = 0, int k_parts = 0, int tile_cols = 0)
        {
            W4A16Route r;
            if (M <= 0 || N <= 0 || K < 128 || (K & 127) || num_cu < 1)
                return r;
            const int n_rows = gate ? 2 * N : N; // weight rows
            const bool any = path == 0, rows_family = any || path == 4, skinny_family = any || path == 2;
            const size_t rstd_bytes = rms ? align256((size_t)M * sizeof(float)) : 0;
            const size_t xn_bytes = rms ? align256((size_t)M * K * 2) : 0;
            if (path != 3)
            {
                // the row-streaming kernels apply prologue and epilogue themselves: one launch, no scratch memory
                if (rows_family && plan_w4a16_rows(M, N, K, num_cu, 0, gate).seg != 0)
                    return r.kind = W4A16Route::ROWS, r.rms_bytes = rstd_bytes, r;
                // (K = 8192 at 8 .. 16 rows: over two ranges of K, see w4a16_mrows_split -- not with SiLU-gate, whose two halves
                // the reduction would have to pair, nor with RMSNorm, which the single launch folds in without a pre-pass)
                const bool two_ranges = !gate && !rms && K == 8192 && M >= 8 && M <= 16 && w4a16_mrows_split(M, n_rows, K, num_cu).ranges > 1;
                if (rows_family && M > 1 && !two_ranges &&
                    (any ? w4a16_mrows_preferred(M, N, K, num_cu, gate) : w4a16_mrows_fits(M, N, K, num_cu, gate)))
                    return r.kind = W4A16Route::MROWS, r.rms_bytes = rstd_bytes, r;
                // the MFMA GEMV kernel writes plain products: an epilogue that cannot work in place (the [M, 2N] gate | up
                // pair, a residual that is the output buffer) reads them from scratch memory
                if (skinny_family && M <= 16 && w4a16_skinny_fits(M, n_rows, K))
                {
                    r.kind = W4A16Route::SKINNY;
                    r.via_scratch = gate || in_place_residual;
                    r.partial_bytes = r.via_scratch ? align256((size_t)M * n_rows * 2) : 0;
                    r.rms_bytes = xn_bytes;
                    return r;
                }
                // more activations than one workgroup holds: ranges of K, fp32 sums per range, and the reduction pass
                // (K above 8192 in multiples of 256: the row-streaming MFMA kernel, otherwise the split-K one)
                if (rows_family && (r.ksplits = w4a16_mrows_split(M, n_rows, K, num_cu).ranges) > 0)
                {
                    r.kind = W4A16Route::MROWS_SPLIT;
                    r.partial_bytes = align256((size_t)r.ksplits * M * n_rows * sizeof(float));
                    r.rms_bytes = rstd_bytes;
                    return r;
                }
                if (skinny_family && (r.ksplits = w4a16_skinny_ksplits(M, n_rows, K)) > 0)
                {
                    r.kind = W4A16Route::SKINNY_SPLIT;
                    r.partial_bytes = align256((size_t)r.ksplits * M * n_rows * sizeof(float));
                    r.rms_bytes = xn_bytes;
                    return r;
                }
                r.ksplits = 0;
                if (!any)
                    return r;
            }
            r.kind = W4A16Route::TILE;
            r.plan = plan_w4a16_sk_with(M, N, K, gate, num_cu, tile_rows, k_parts, tile_cols);
            r.partial_bytes = r.plan.bytes();
            r.rms_bytes = rstd_bytes;
            return r;
        }

        inline bool w4a16_variant_fits(int M, int N, int K, int variant, int num_cu)
        {
            if (M <= 0 || N <= 0 || K < 128 || (K & 127))
                return false;
            if (variant == 1)
                return w4a16_gemv_valu_fits(M, K);
            return variant >= 0 && variant <= 4 && route_w4a16(M, N, K, false, false, false, num_cu, variant).kind != W4A16Route::NONE;
        }
        // nnf_w4a16_gemm: [ partial sums ]
        inline size_t w4a16_gemm(int M, int N, int K, int, int num_cu)
        {
            return route_w4a16(M, N, K, false, false, false, num_cu).partial_bytes;
        }
        // nnf_w4a16_gemm_fused: [ RMSNorm scratch ][ partial sums ], whichever of the optional parts the call uses
        inline size_t w4a16_gemm_fused(int M, int N, int K, int, int act, int num_cu = PLAN_CUS)
        {
            // (with and without the RMSNorm prologue, with the residual in place or not: the routes differ -- 8 .. 16 rows
            // at K = 8192 run over two ranges of K only without the prologue)
            const bool gate = act == 1;
            size_t most = 0;
            for (int rms = 0; rms < 2; ++rms)
                for (int in_place = 0; in_place < (gate ? 1 : 2); ++in_place)
                {
                    const W4A16Route r = route_w4a16(M, N, K, gate, rms != 0, in_place != 0, num_cu);
                    const size_t bytes = r.rms_bytes + r.partial_bytes;
                    most = bytes > most ? bytes : most;
                }
            return most;
        }
        // nnf_fused_mlp_w4a16: [ RMSNorm scratch of the first product ][ h: M x I fp16 ][ partial sums of either product ]
        inline size_t fused_mlp_h_offset(int M, int H, int I, int num_cu = PLAN_CUS)
        {
            return route_w4a16(M, I, H, true, true, false, num_cu).rms_bytes;
        }
        inline size_t fused_mlp_partial_offset(int M, int H, int I, int num_cu = PLAN_CUS)
        {
            return fused_mlp_h_offset(M, H, I, num_cu) + align256((size_t)M * I * 2);
        }
        inline size_t fused_mlp_w4a16(int M, int H, int I, int, int num_cu = PLAN_CUS)
        {
            if (M <= 0 || I <= 0 || H < 128 || I < 128)
                return 0;
            const size_t a = route_w4a16(M, I, H, true, true, false, num_cu).partial_bytes;
            // (the second product's residual x may be the output buffer itself)
            const size_t b = route_w4a16(M, H, I, false, false, false, num_cu).partial_bytes;
            const size_t c = route_w4a16(M, H, I, false, false, true, num_cu).partial_bytes;
            const size_t bc = b > c ? b : c;
            return fused_mlp_partial_offset(M, H, I, num_cu) + (a > bc ? a : bc);
        }
    } // namespace workspace
} // namespace nnf
