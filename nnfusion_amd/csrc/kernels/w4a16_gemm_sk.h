// fp16 x int4 (g128) MFMA tile GEMM for gfx950: four wavefronts side by side along N, work split evenly
// over the CUs.
//
//   Y[M,N] = epilogue( prologue(A)[M,K] . ((Wq - zp) * S)^T )
//
// Replaces the cublasSgemm/cublasHgemm call that the reference's cuda::Dot emits
// (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:128-205, 271-363) for a weight-quantized Dot
// with transpose_B, plus the element-wise kernels around it (RMSNorm ahead of it, bias / residual /
// SiLU(gate) * up behind it; fusion precedent: cuda_gpu/kernels/elementwise_fused.cpp:43-288,
// matmuladd.cpp:29-93).
//
// Two things bound a quantized GEMM on this chip besides the matrix cores.  The chip is power managed:
// every byte of fresh data moved next to an MFMA lowers the clock the MFMAs run at.  And with the
// accumulators of a 256 x 256 tile in registers there is one wavefront per SIMD, whose vector, LDS and
// memory instructions are issued between its own MFMAs and not under them.  The structure therefore
// minimises traffic and instructions per MFMA:
//   * One workgroup = four wavefronts (one per SIMD, up to 512 registers each) over a (TM*32) x (TN*128)
//     tile, each wavefront owning all TM*32 rows of a strip of TN*32 columns (TM x TN MFMA tiles of
//     32x32x16).  A weight belongs to exactly one wavefront: it is unpacked once per workgroup (16 VALU
//     operations per 8 weights, feeding TM MFMAs each), not once per wavefront row.
//   * A lane owns one weight row of each of its column tiles and one half of every 64-wide K step, and holds the
//     weights of one "superstep" of 256 k (two quantization groups, four K steps) in registers at a time: 4 x 16
//     bytes per column tile.  The largest tile (256 x 256) fetches them straight into registers, two register sets,
//     superstep s+1 requested while s is multiplied.  Such a load touches 32 bytes of each of 32 rows; measured
//     with the same bytes fetched as whole lines, loads of that shape cost the memory pipeline about four times
//     what loads of whole 128-byte lines cost it, and with smaller tiles -- fewer MFMAs per load -- the K loop
//     waits for them.  Every other tile therefore moves a superstep's 32 x 128 bytes per column tile global -> LDS
//     (four loads of 8 whole rows, global_load_lds_dwordx4, into an area of the wavefront's own: no barrier) one
//     superstep ahead, and from there into the registers (four ds_read_b128 per column tile) at the last barrier
//     of the superstep before, under that quarter's MFMAs.  The group scales are two 2-byte loads per row and
//     superstep into registers in both forms.
//   * The activations go global -> LDS asynchronously (global_load_lds_dwordx4, no register staging)
//     into a ring of three stages of BK = 64; the loads for K step kt+3 are issued from the barrier of
//     step kt on, a quarter of them per quarter step.
//   * One barrier per K step, placed ahead of the step's LAST quarter: at that point every fragment of
//     the step is in registers, so the stage can be refilled at once, and the first fragments of the
//     next step are read while the last MFMAs of this one run.
//   * The instruction stream is laid out in regions of a few MFMAs + their fragment reads + a share of
//     the unpacking + at most a few loads, so that no queue (LDS, address unit) sees a burst.  Every load
//     has a scalar base and a 32-bit lane offset that never changes, and the waits on the loads into LDS
//     and on the fragment reads are counted by hand (the compiler's own would drain everything in flight).
//   * The workgroups of a launch split the flat list of (tile, superstep) units evenly ("stream-K"): a
//     launch has one workgroup per CU with the same amount of work, whatever the tile count (the plan launches one
//     workgroup per tile instead where the tiles fill at least half of the CUs and K is short: sharing tiles costs
//     more than the idle CUs there).  A
//     workgroup that covers only part of a tile's K range writes its fp32 sums to the workspace in
//     register order (1 KiB per store instruction); a second, small launch adds the parts of such tiles
//     in K order and runs their epilogue, on all CUs (one CU would need tens of microseconds to pull the
//     parts of a tile through its own registers).  Tiles with a single owner are finished here.
//     Given two zeroed words per tile (SkGemmParams::sync) the second launch is not needed: the workgroups that
//     share a tile count their arrivals there and each adds up and finishes its share of the tile's 32-row blocks
//     once all have arrived, in the same K order (same bits as the second launch gives).
//   * Epilogues round the way the unfused graph would: the GEMM result to fp16 first, then the
//     element-wise operation in fp32, then fp16 again.  RMSNorm is folded in without materialising the
//     normalised activations: gamma[k] multiplies the weights as they are unpacked, rstd[m] multiplies the
//     fp32 row sums.  rstd[] comes from a small pre-pass over A, or (SkGemmParams::rstd_out, one-launch form) from
//     the launch itself: every workgroup adds up the squares of a few rows before its first tile, and an
//     epilogue waits (bounded) until all have.
#pragma once

#include "nnf_device.h"
#include "nnf_launch.h"

namespace nnf
{
    struct SkGemmParams
    {
        const half_t* A;
        const uint8_t* Wq;
        const half_t* S;
        half_t* Y;
        int M, N, K, zp;        // N = output columns
        int ldy;                // row stride of Y
        int up_row_offset;      // GATE: weight row of the up projection that pairs with gate row 0
        const half_t* bias;     // BIAS: [N]
        const half_t* residual; // RESID: [M, ldy]
        const half_t* gamma;    // RMS: [K]
        const float* rstd;      // RMS: [M]
        float* partial;         // slots of BM x BN fp32: workgroup v's first segment at slot v, a later one at grid + v
        size_t partial_bytes;   // all slots
        int tiles_m, tiles_n;
        int supersteps;         // per tile: ceil(K / 256)
        long long units;        // tiles_m * tiles_n * supersteps
        const uint8_t* zps;     // QG != 0: zero points, u8 [N, K / group / 2] (even group in the low nibble), or null: zp
        // One launch instead of two: two words per tile, all zero when the launch starts and zero again when it ends.
        // Non-null: the workgroups that share a tile add its parts up themselves (sk_reduce_shared_tile below) and no
        // second launch follows.
        uint32_t* sync;
        int spin_limit;         // polls of a tile's arrival count before a workgroup leaves its share to the last arriver
        // RMS without a pass of its own: non-null, the launch computes rstd[] itself -- workgroup v the rows v, v + grid,
        // ... before its first tile, into `rstd_out` (= rstd) -- and counts in rstd_sync[0] the workgroups that have done
        // so, in rstd_sync[1] those that have ended (two more words, zero at the start, zero again at the end).
        float* rstd_out;
        uint32_t* rstd_sync;
        float rms_eps;
        // NNF_SK_TRACE builds only (the measurement probes): 16 time stamps of the 100 MHz clock per workgroup, or null
        unsigned long long* trace;
    };

    // Time stamps inside the GEMM kernel for the measurement probes: compiled in only with NNF_SK_TRACE (the product
    // library is built without it).  Stamp i of workgroup v: thread 0, SkGemmParams::trace[16 v + i].
#ifdef NNF_SK_TRACE
#define NNF_SK_STAMP(i)                                                                                                 \
    do                                                                                                                  \
    {                                                                                                                   \
        if (p.trace && threadIdx.x == 0)                                                                                \
            p.trace[(size_t)v * 16 + (i)] = __builtin_amdgcn_s_memrealtime();                                          \
    } while (0)
#else
#define NNF_SK_STAMP(i)                                                                                                 \
    do                                                                                                                  \
    {                                                                                                                   \
    } while (0)
#endif

    namespace gemm_sk
    {
        constexpr int BK = 64;
        constexpr int WAVES = 4;
        constexpr int THREADS = WAVES * 64;
        constexpr int STAGES = 3;

        template <int TM, int TN>
        struct Tile
        {
            static constexpr int BM = TM * 32;
            static constexpr int BN = WAVES * TN * 32; // weight rows per tile (GATE: half gate, half up rows)
            static constexpr int A_TILE_BYTES = BM * BK * 2;
            // per wavefront 256 bytes: (RMS) the step's 64 gamma values twice over
            static constexpr int CONST_BYTES = WAVES * 256;
            static constexpr int STAGE_BYTES = A_TILE_BYTES + CONST_BYTES;
            // the epilogue turns the results through a private piece of the ring per wavefront
            static constexpr int EPILOGUE_BYTES = WAVES * (TM >= 2 ? 2 : 1) * 32 * (TN * 64 + 16);
            // Weights through LDS (see the kernel): every tile but the largest, whose K step is long enough for the loads
            // it has and which has the least LDS bandwidth to spare (M = 4096, N = K = 8192: 2 % slower that way;
            // M = 1024 on 256 x 128 tiles: 3 % faster; 128-row tiles: 3 - 7 % faster).  Behind the ring: per wavefront
            // and column tile the 32 x 128 bytes of the next superstep
            static constexpr bool W_VIA_LDS = !(TM == 8 && TN >= 2);
            static constexpr int W_LDS_OFFSET = STAGES * STAGE_BYTES > EPILOGUE_BYTES ? STAGES * STAGE_BYTES : EPILOGUE_BYTES;
            static constexpr int W_LDS_BYTES = W_VIA_LDS ? WAVES * TN * 4096 : 0;
            static constexpr int LDS_BYTES = W_LDS_OFFSET + W_LDS_BYTES;
            static constexpr size_t SLOT_FLOATS = (size_t)BM * BN;
        };

        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

        // `grid` workgroups split `units` units as [v * units / grid, (v + 1) * units / grid)
        // (A workgroup whose share spans two tiles parks the first tile's part in the middle of the launch, where the
        // acknowledgement of its device-scope stores takes about 5 us against 2-3 us at the end of the launch.  Issuing the
        // next segment's first loads ahead of those stores was tried: the acknowledgement, not the loads, is what the
        // workgroup waits for, and nothing was gained.  Stores and loads at the scope of one XCD's L2 instead of the device
        // -- valid only among workgroups known to sit on one XCD -- were timed in the measurement probe: acknowledged in 2 us
        // there, but the last workgroup of the launch ended less than a microsecond earlier.)
        // (Shares weighted by what a second K loop in a workgroup costs -- its first loads, parking the part it leaves
        // behind: about one and a half units -- were tried: with whole units to deal out the longest share stays the same
        // for the MLP block's products, and a table of bounds in the kernel arguments made every launch slower.)
        __host__ __device__ inline long long first_unit_of(int v, long long units, int grid)
        {
            return ((long long)v * units) / grid;
        }
        // the workgroup that owns unit x
        __host__ __device__ inline int owner_of_unit(long long x, long long units, int grid)
        {
            return (int)(((x + 1) * grid - 1) / units);
        }

        // Which loads a wavefront issues where.  A K step has four quarters of TM x TN MFMAs; step kt is of type
        // T = kt mod 4 (its place in the superstep).
        //   * The TM activation loads (+ gamma with RMS) for step kt+3 go out in four positions: position 0 in
        //     quarter 3 of step kt (right behind the barrier that frees the stage), positions 1 .. 3 in quarters
        //     0 .. 2 of step kt+1.
        //   * The NW loads (four of weights, the others scales and zero points) per column tile for the next superstep
        //     go out in quarters 0 .. 2 of step T = w_step(tile), ahead of that quarter's activation loads.
        //     (NW: loads per column tile and superstep, weights and scales)
        template <int TM, int TN, bool RMS, int NW>
        struct Sched
        {
            static constexpr int a_pos(int i) { return (i * 4) / TM; }
            static constexpr int a_loads_at(int pos)
            {
                int n = (RMS && pos == 0) ? 1 : 0;
                for (int i = 0; i < TM; ++i)
                    n += a_pos(i) == pos ? 1 : 0;
                return n;
            }
            static constexpr int a_loads_total() { return TM + (RMS ? 1 : 0); }
            // two tiles in the first step where there are four: everything has been asked for by the end of step 2
            static constexpr int w_step(int j) { return TN <= 3 ? j : (j < 2 ? 0 : j - 1); }
            static constexpr int w_loads_in_step(int T)
            {
                int n = 0;
                for (int j = 0; j < TN; ++j)
                    n += w_step(j) == T ? NW : 0;
                return n;
            }
            // the step's weight loads number [w_begin(T, Q), w_begin(T, Q + 1)) go out in quarter Q (0 .. 2)
            static constexpr int w_begin(int T, int Q) { return Q * w_loads_in_step(T) / 3; }
            // the x-th weight load of a step of type T: column tile and which of its six loads
            static constexpr int w_tile(int T, int x)
            {
                int seen = 0;
                for (int j = 0; j < TN; ++j)
                    if (w_step(j) == T)
                    {
                        if (x < seen + NW)
                            return j;
                        seen += NW;
                    }
                return -1;
            }
            static constexpr int w_which(int x) { return x % NW; }
            static constexpr int loads_at(int T, int Q)
            {
                return Q == 3 ? a_loads_at(0) : (w_begin(T, Q + 1) - w_begin(T, Q)) + a_loads_at(Q + 1);
            }
            // loads issued behind the last activation load for step kt+1 up to the wait that opens quarter 3 of step
            // kt (vector-memory operations complete in order): what may still be outstanding there
            static constexpr int later(int T)
            {
                const int Tp = (T + 3) & 3;
                const int lp = a_pos(TM - 1); // 0: the last one went out in quarter 3 of step kt-2, p: in quarter p-1 of step kt-1
                int n = 0;
                for (int Q = lp; Q < 3; ++Q)
                    n += loads_at(Tp, Q);
                n += loads_at(Tp, 3);
                for (int Q = 0; Q < 3; ++Q)
                    n += loads_at(T, Q);
                // the last step of a superstep also wants the next superstep's weights: everything but the
                // activation loads issued since quarter 3 of step 2
                if (T == 3 && n > a_loads_total())
                    n = a_loads_total();
                return n;
            }
        };


        // Every load is one the compiler can see, so that its own wait insertion protects the registers they fill
        // (also against copies its register allocator may place): global -> LDS through the builtin, weights and
        // scales as ordinary loads.  Two things keep them cheap.  Scalar base addresses pass through an empty asm
        // statement: the compiler then keeps them in scalar registers; lane offsets are redefined where they are
        // used: the widening to 64 bits stays next to the load and is folded into it (scalar base + 32-bit lane
        // offset), instead of being hoisted out of the loop as a register pair.  And the workgroup barrier is
        // written as assembly: ahead of a barrier it knows, the compiler waits for every load in flight.
        __device__ __forceinline__ const uint8_t* scalar_base(const uint8_t* ptr)
        {
            asm("" : "+s"(ptr));
            return ptr;
        }
        __device__ __forceinline__ uint32_t here(uint32_t off)
        {
            asm volatile("" : "+v"(off));
            return off;
        }
        typedef const void __attribute__((address_space(1))) * global_ptr;
        typedef void __attribute__((address_space(3))) * lds_ptr;
        __device__ __forceinline__ void workgroup_barrier()
        {
            asm volatile("s_barrier" ::: "memory");
        }

        // regions per quarter and fragments per region
        constexpr int regions_of(int TM) { return TM < 4 ? TM : 4; }

        // Parked sums that other workgroups of the SAME launch read (SkGemmParams::sync): stores and loads at device
        // scope (the sc1 bit), i.e. written through to, and read from, the level of the memory system that all eight
        // L2s of the chip agree on.  A release / acquire fence pair would do the same for ordinary accesses, but on
        // this chip such a fence writes back / invalidates a whole L2 under the 32 CUs that share it: with fences
        // the one-launch form measured twice as slow as the two-launch form.  Buffer instructions, because their
        // intrinsics take the cache policy as an argument and the compiler tracks them like any other load (a load
        // written as inline assembly would land in registers the compiler may have given away again).
        typedef __amdgpu_buffer_rsrc_t buffer_t;
        constexpr int DEVICE_SCOPE = 16; // sc1
        __device__ __forceinline__ buffer_t parked_buffer(float* base, size_t bytes)
        {
            // raw buffer over [base, base + bytes): accesses beyond it read zero / are dropped
            return __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : bytes), 0x00020000);
        }
        __device__ __forceinline__ void store_device_scope(buffer_t buf, uint32_t byte_offset, const floatx4& v)
        {
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, v), buf, (int)byte_offset, 0, DEVICE_SCOPE);
        }
        __device__ __forceinline__ floatx4 load_device_scope(buffer_t buf, uint32_t byte_offset)
        {
            return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(buf, (int)byte_offset, 0, DEVICE_SCOPE));
        }
        // every vector-memory operation of this wavefront is complete (stores: acknowledged at their scope)
        __device__ __forceinline__ void wait_vector_memory()
        {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    } // namespace gemm_sk

    // Epilogue of one round (ROUND_TM blocks of 32 rows) of a wavefront's strip of a tile.  Lane (m = l32, h) holds, in
    // element e of MFMA tile (ii, j), column n = 8*(e/4) + 4*h + (e%4) of row ii*32 + m.  The sums are rounded (GATE:
    // combined) in registers, turned through a private piece of LDS (`region`: sk_region_bytes) and finished as whole rows of the strip, 16 bytes
    // (8 columns) per lane: bias, residual, store.  Rounding as the unfused graph would: the GEMM result to fp16 first,
    // then the element-wise operation in fp32, then fp16 again.
    // bytes of LDS sk_finish_round uses per wavefront
    template <int TM, int TN, bool GATE>
    constexpr int sk_region_bytes()
    {
        return (TM >= 2 ? 2 : 1) * 32 * ((GATE ? TN / 2 : TN) * 64 + 16);
    }

    template <int TM, int TN, bool GATE, bool BIAS, bool RESID, bool RMS>
    __device__ __forceinline__ void sk_finish_round(const SkGemmParams& p, const floatx16 (&c)[TM >= 2 ? 2 : 1][TN], int r, int m0, int n0,
                                                    uint8_t* region, int wave, int lane)
    {
        constexpr int OUT_TN = GATE ? TN / 2 : TN;
        constexpr int ROUND_TM = TM >= 2 ? 2 : 1;
        constexpr int PITCH = OUT_TN * 64 + 16; // bytes per staged row (padding spreads the banks)
        constexpr int LANES_PER_ROW = OUT_TN * 4, ROWS_PER_READ = 64 / LANES_PER_ROW;
        const int l32 = lane & 31, h = lane >> 5;
        const int n_wave = n0 + wave * (OUT_TN * 32);
        const int piece = lane % LANES_PER_ROW;
        const int n_lane = n_wave + piece * 8; // first of this lane's 8 columns in the row phase
        bool vec = ((p.N & 7) == 0) && ((p.ldy & 7) == 0) && ((reinterpret_cast<uintptr_t>(p.Y) & 15) == 0);
        if (RESID)
            vec = vec && ((reinterpret_cast<uintptr_t>(p.residual) & 15) == 0);
        float bias[8];
        if (BIAS)
        {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                bias[k] = (float)p.bias[min(n_lane + k, p.N - 1)];
        }
#pragma unroll
        for (int ii = 0; ii < ROUND_TM; ++ii)
        {
            const int i = r * ROUND_TM + ii;
            float rs = 1.0f;
            if (RMS) // (device scope: other workgroups of this launch may have written it)
                rs = __hip_atomic_load(p.rstd + min(m0 + i * 32 + l32, p.M - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int j = 0; j < OUT_TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    half4_t y;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                    {
                        if (GATE)
                        {
                            const float gt = (float)(half_t)(RMS ? c[ii][j][4 * g + k] * rs : c[ii][j][4 * g + k]);
                            const float up =
                                (float)(half_t)(RMS ? c[ii][j + TN / 2][4 * g + k] * rs : c[ii][j + TN / 2][4 * g + k]);
                            y[k] = (half_t)(gt * (1.0f / (1.0f + __expf(-gt))) * up);
                        }
                        else
                        {
                            y[k] = (half_t)(RMS ? c[ii][j][4 * g + k] * rs : c[ii][j][4 * g + k]);
                        }
                    }
                    *reinterpret_cast<half4_t*>(region + (ii * 32 + l32) * PITCH + (j * 32 + 8 * g + 4 * h) * 2) = y;
                }
        }
        // LDS operations of one wavefront execute in order: no barrier around the private region
#pragma unroll
        for (int it = 0; it < ROUND_TM * 32 / ROWS_PER_READ; ++it)
        {
            const int row = it * ROWS_PER_READ + lane / LANES_PER_ROW;
            half8_t o = *reinterpret_cast<const half8_t*>(region + row * PITCH + piece * 16);
            const int m = m0 + r * (ROUND_TM * 32) + row;
            if (m >= p.M || n_lane >= p.N)
                continue;
            const size_t at = (size_t)m * p.ldy + n_lane;
            if (BIAS)
            {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    o[k] = (half_t)((float)o[k] + bias[k]);
            }
            if (RESID)
            {
                half8_t res;
                if (vec)
                    res = *reinterpret_cast<const half8_t*>(p.residual + at);
                else
                    for (int k = 0; k < 8; ++k)
                        res[k] = p.residual[n_lane + k < p.N ? at + k : at];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    o[k] = (half_t)((float)o[k] + (float)res[k]);
            }
            if (vec)
                *reinterpret_cast<half8_t*>(p.Y + at) = o;
            else
                for (int k = 0; k < 8; ++k)
                    if (n_lane + k < p.N)
                        p.Y[at + k] = o[k];
        }
    }

    // Block `r` (32 rows) of strip `wave` of a tile that `n_seg` workgroups (v_first, v_first + 1, ...) of a launch of
    // `gemm_grid` worked on: adds their parked parts in K order, eight in flight, and finishes the block (epilogue,
    // stores).  Used by the second launch and, with SkGemmParams::sync, by the GEMM's own workgroups: same order, same bits.
    // Where a shared tile's parts lie and what its rows and columns are: what sk_request_parts / sk_finish_block need
    struct SkSharedTile
    {
        int tile, v_first, n_seg;
        bool first_is_second_slot; // the first owner parked this tile in its second slot (its range began in an earlier tile)
    };
    // Parts of a block kept in flight at once (16 TN registers each).  SAME_LAUNCH: inside the GEMM kernel, with its
    // accumulation registers still set aside, and (sk_loads_ahead) two blocks' worth of them in flight.
    template <int TM, int TN>
    constexpr bool sk_loads_ahead()
    {
        return TM * TN <= 8;
    }
    template <int TM, int TN, bool SAME_LAUNCH>
    struct SkPartsInFlight
    {
        static constexpr int D = !SAME_LAUNCH ? 8 : (sk_loads_ahead<TM, TN>() && TN >= 2) ? 3 : 4;
        floatx4 v[D][TN][4]; // [part][column tile][quarter of its 16 elements]
    };
    // Asks for parts sg0 .. sg0 + D - 1 (clamped to the last) of block `r` (32 rows) of strip `wave` of a shared tile.
    // SAME_LAUNCH: the parts were parked by other workgroups of the launch that is still running (device-scope loads).
    template <int TM, int TN, bool SAME_LAUNCH>
    __device__ __forceinline__ void sk_request_parts(SkPartsInFlight<TM, TN, SAME_LAUNCH>& x, const SkGemmParams& p,
                                                     int gemm_grid, const SkSharedTile& t, int r, int sg0, int tid)
    {
        using namespace gemm_sk;
        using T = Tile<TM, TN>;
        constexpr int D = SkPartsInFlight<TM, TN, SAME_LAUNCH>::D;
        buffer_t parked;
        if constexpr (SAME_LAUNCH)
            parked = parked_buffer(p.partial, p.partial_bytes);
#pragma unroll
        for (int d = 0; d < D; ++d)
        {
            const int sg = min(sg0 + d, t.n_seg - 1);
            const size_t first_float =
                ((size_t)(t.v_first + sg) + ((sg == 0 && t.first_is_second_slot) ? (size_t)gemm_grid : 0)) * T::SLOT_FLOATS + (size_t)tid * 4;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                {
                    const size_t at = first_float + (size_t)(((r * TN + j) * 4 + q) * THREADS * 4);
                    if constexpr (SAME_LAUNCH)
                        x.v[d][j][q] = load_device_scope(parked, (uint32_t)(at * sizeof(float)));
                    else
                        x.v[d][j][q] = *reinterpret_cast<const floatx4*>(p.partial + at);
                }
        }
    }
    // Block `r` (32 rows) of strip `wave` of a tile that t.n_seg workgroups (t.v_first, t.v_first + 1, ...) of a launch of
    // `gemm_grid` worked on: adds their parked parts in K order -- the first ones have been asked for into `x` -- and
    // finishes the block (epilogue, stores).  Used by the second launch and, with SkGemmParams::sync, by the GEMM's own
    // workgroups: same order, same bits.
    template <int TM, int TN, bool GATE, bool BIAS, bool RESID, bool RMS, bool SAME_LAUNCH>
    __device__ __forceinline__ void sk_finish_block(SkPartsInFlight<TM, TN, SAME_LAUNCH>& x, const SkGemmParams& p,
                                                    int gemm_grid, const SkSharedTile& t, int r, uint8_t* stage, int wave, int lane)
    {
        using namespace gemm_sk;
        using T = Tile<TM, TN>;
        constexpr int BN_OUT = GATE ? T::BN / 2 : T::BN;
        constexpr int D = SkPartsInFlight<TM, TN, SAME_LAUNCH>::D;
        int tm, tn;
        {
            constexpr int GM = 4;
            const int per_group = GM * p.tiles_n;
            const int g = t.tile / per_group;
            const int first_m = g * GM;
            const int gm = min(GM, p.tiles_m - first_m);
            const int rr = t.tile - g * per_group;
            tm = first_m + rr % gm;
            tn = rr / gm;
        }
        const int m0 = tm * T::BM, n0 = tn * BN_OUT;
        floatx16 c[1][TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                c[0][j][e] = 0.f;
        for (int sg0 = 0; sg0 < t.n_seg; sg0 += D)
        {
            if (sg0 > 0)
                sk_request_parts<TM, TN, SAME_LAUNCH>(x, p, gemm_grid, t, r, sg0, wave * 64 + lane);
#pragma unroll
            for (int d = 0; d < D; ++d)
                if (sg0 + d < t.n_seg)
                {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                        {
                            c[0][j][4 * q] += x.v[d][j][q].x;
                            c[0][j][4 * q + 1] += x.v[d][j][q].y;
                            c[0][j][4 * q + 2] += x.v[d][j][q].z;
                            c[0][j][4 * q + 3] += x.v[d][j][q].w;
                        }
                }
        }
        sk_finish_round<1, TN, GATE, BIAS, RESID, RMS>(p, c, r, m0, n0, stage, wave, lane);
    }

    // rstd[m] = rsqrt(mean_k(A[m, k]^2) + eps) for rows first, first + step, ... < end by the 256 threads of a workgroup
    // (the summation order of the pre-pass kernel, rms_rstd_kernel: same bits), stored at device scope; complete for
    // every thread of the workgroup on return.  part: four floats of LDS.
    __device__ __forceinline__ void sk_rstd_rows(const SkGemmParams& p, int first, int end, int step, float* part, int tid)
    {
        const int units = p.K >> 3;
        for (int m = first; m < end; m += step)
        {
            const uintx4* row = reinterpret_cast<const uintx4*>(p.A + (size_t)m * p.K);
            float ss = 0.f;
            for (int i = tid; i < units; i += gemm_sk::THREADS)
            {
                const uintx4 v = row[i];
                const uint32_t vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const half2_t hh = as_half2(vv[j]);
                    ss += (float)hh.x * (float)hh.x + (float)hh.y * (float)hh.y;
                }
            }
            ss = wave_sum(ss);
            if ((tid & 63) == 0)
                part[tid >> 6] = ss;
            __syncthreads();
            if (tid == 0)
                __hip_atomic_store(p.rstd_out + m, 1.0f / __builtin_sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)p.K + p.rms_eps),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
        }
        gemm_sk::wait_vector_memory();
        __syncthreads();
    }

    // SkGemmParams::sync, word 0 of a tile: bits 0 .. 15 count the workgroups that have parked their part of it, bits
    // 16 .. 23 mark the 32-row blocks whose owner stopped waiting (the last arriver takes them over); word 1 counts the
    // blocks that are finished: whoever finishes the last one sets both words to zero again.
    // Thread 0 of a workgroup that has arrived (`old`: the word as its own arrival found it) and owns the blocks
    // `own_mask`: the blocks to add up and finish now.  Waits at most `spin_limit` polls for the other arrivals.
    __device__ __forceinline__ uint32_t sk_blocks_to_finish(uint32_t* state, uint32_t old, int n_seg, uint32_t own_mask, int spin_limit)
    {
        if ((old & 0xFFFFu) == (uint32_t)(n_seg - 1))
            return own_mask | ((old >> 16) & 0xFFu);
        if (own_mask == 0)
            return 0;
        for (int polls = 0;; ++polls)
        {
            const uint32_t s = __hip_atomic_load(state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((s & 0xFFFFu) == (uint32_t)n_seg)
                return own_mask;
            if (polls >= spin_limit)
            {
                // hand the blocks over -- unless an arrival gets in first (the exchange fails: look again)
                uint32_t expected = s;
                if (__hip_atomic_compare_exchange_strong(state, &expected, s | (own_mask << 16), __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT))
                    return 0;
                continue;
            }
            __builtin_amdgcn_s_sleep(2);
        }
    }

    // QG = 0: groups of 128, the zero point p.zp.  QG = 5, 6, 7: groups of 2^QG and, with p.zps, a zero point per
    // (row, group); K a multiple of 256.  A lane's 32 weights of a K step lie in one group whatever its size: per column
    // tile and superstep it fetches the 256 / group scales of its row in one load (4, 8 or 16 bytes) and the byte(s) that
    // hold their zero points in another (1, 2 or 4 bytes; without p.zps: the scales again, unused) -- six loads per
    // column tile as for QG = 0, on the same schedule -- and keeps a scale and the pair -(1024 + z), -(64 + z) per K step.
    template <int TM, int TN, bool GATE, bool BIAS, bool RESID, bool RMS, int QG = 0>
    __global__ __launch_bounds__(256, 1) void w4a16_gemm_sk_kernel(const half_t* __restrict__ A_first,
                                                                   const uint8_t* __restrict__ Wq_first,
                                                                   const half_t* __restrict__ S_first, long long units_first,
                                                                   int M_first, int N_first, int K_first, int tiles_n_first,
                                                                   int supersteps_first, int grid_first, SkGemmParams p_rest)
    {
        // (what the first loads need, once more as arguments of their own -- launch_sk_kernel passes them: fourteen dwords
        // of scalar arguments arrive in registers with the wavefront, a structure passed by value and the size of the
        // grid are loaded from memory, and the kernel began by waiting for them)
        SkGemmParams p = p_rest;
        p.A = A_first;
        p.Wq = Wq_first;
        p.S = S_first;
        p.units = units_first;
        p.M = M_first;
        p.N = N_first;
        p.K = K_first;
        p.tiles_n = tiles_n_first;
        p.supersteps = supersteps_first;
        using namespace gemm_sk;
        using T = Tile<TM, TN>;
        // loads per column tile and superstep: four of weights; two of scales and zero points, or (the specialised kernel)
        // three of scales, see load_w
        constexpr int NW = QG != 0 ? 6 : 7;
        using SCH = Sched<TM, TN, RMS, NW>;
        static_assert(!(GATE && (BIAS || RESID)), "SiLU-gate is not combined with bias or residual");
        static_assert(TN == 1 || TN == 2 || TN == 4, "column tiles per wavefront");
        static_assert(!GATE || TN >= 2, "gate and up rows are the two halves of a wavefront's column tiles");
        static_assert(QG == 0 || (QG >= 5 && QG <= 7), "groups of 32, 64 or 128");
        constexpr bool QZ = QG != 0;
        constexpr int GSH = QZ ? QG : 7;                    // log2 of the group size
        constexpr int NSC = QZ ? (QG == 7 ? 2 : 4) : 2;     // scales a lane keeps per column tile and superstep
        constexpr int SW = QZ ? (QG == 5 ? 4 : QG == 6 ? 2 : 1) : 3; // registers of scales as loaded
        constexpr int BM = T::BM, BN = T::BN;
        constexpr int A_TILE_BYTES = T::A_TILE_BYTES, STAGE_BYTES = T::STAGE_BYTES;
        constexpr int BN_OUT = GATE ? BN / 2 : BN;
        constexpr int NREG = regions_of(TM); // regions per quarter
        constexpr int FPR = TM / NREG;       // activation fragments per region
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        // volatile: the vector move has to stay here, where every lane is active
        uint32_t MASK, MAGIC, SEL[4];
        asm volatile("v_mov_b32 %0, 0x54006400" : "=v"(MAGIC));
        asm volatile("s_mov_b32 %0, 0x00F0000F" : "=s"(MASK));
        asm volatile("s_mov_b32 %0, 0x0c000c00" : "=s"(SEL[0]));
        asm volatile("s_mov_b32 %0, 0x0c010c01" : "=s"(SEL[1]));
        asm volatile("s_mov_b32 %0, 0x0c020c02" : "=s"(SEL[2]));
        asm volatile("s_mov_b32 %0, 0x0c030c03" : "=s"(SEL[3]));
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int l32 = lane & 31, h = lane >> 5;
        const int K = p.K;
        const int G = K >> GSH;
        const bool g_even = !(G & 1);
        const int SS = p.supersteps;
        const int grid = grid_first; // = gridDim.x
        const uint32_t lds0 = lds_address(smem);

        // workgroup ids are dealt round-robin to the 8 XCDs: number the workgroups so that an XCD (own L2) holds a
        // contiguous run of them, i.e. of units, i.e. of tiles
        int v;
        {
            const int pid = (int)blockIdx.x;
            const int per_xcd = (grid + 7) >> 3;
            const int full = grid - (per_xcd - 1) * 8;
            const int xcd = pid & 7, idx = pid >> 3;
            v = (xcd < full) ? xcd * per_xcd + idx : full * per_xcd + (xcd - full) * (per_xcd - 1) + idx;
        }
        const long long u_begin = first_unit_of(v, p.units, grid), u_end = first_unit_of(v + 1, p.units, grid);
        NNF_SK_STAMP(0); // the workgroup runs

        // ---- (rstd_out) RMSNorm's rstd[] inside this launch: this workgroup's rows now, counted in once they are
        // visible to every CU; an epilogue looks at the count before it reads rstd[] (ensure_rstd) ------------------
        __shared__ float rstd_part[4];
        __shared__ uint32_t rstd_note;
        bool rstd_ok = true; // (uniform) rstd[] is known to be complete
        if constexpr (RMS)
        {
            if (p.rstd_out)
            {
                rstd_ok = false;
                sk_rstd_rows(p, v, p.M, grid, rstd_part, tid);
                if (tid == 0)
                    atomicAdd(p.rstd_sync, 1u);
            }
        }
        // before an epilogue of rows [m_first, m_end): every workgroup has counted itself in -- or, when the (bounded)
        // wait for that runs out, the rows are computed here (the same values, whoever stores them)
        auto ensure_rstd = [&](int m_first, int m_end) {
            if constexpr (RMS)
            {
                if (rstd_ok)
                    return;
                if (tid == 0)
                {
                    uint32_t seen = 0u;
                    for (int polls = 0; polls < p.spin_limit; ++polls)
                    {
                        seen = __hip_atomic_load(p.rstd_sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (seen == (uint32_t)grid)
                            break;
                        __builtin_amdgcn_s_sleep(2);
                    }
                    rstd_note = seen == (uint32_t)grid ? 1u : 0u;
                }
                __syncthreads();
                rstd_ok = rstd_note != 0u;
                __syncthreads();
                if (!rstd_ok)
                    sk_rstd_rows(p, m_first, min(m_end, p.M), 1, rstd_part, tid);
            }
        };

        // (q - zp) from (1024 + q_even, 64 + q_odd): exact
        const half2_t dq_add = half2_t{(half_t)(-(1024.0f + (float)p.zp)), (half_t)(-(64.0f + (float)p.zp))};

        // per-lane fragment addresses within a stage: row l32 of every 32-row block shares its swizzle
        uint32_t a_rd[4]; // quarter s: piece (4h + s) ^ swizzle of row l32
#pragma unroll
        for (int s = 0; s < 4; ++s)
            a_rd[s] = lds0 + (uint32_t)(l32 * 128 + ((((h << 2) + s) ^ ((l32 >> 1) & 7)) << 4));
        // gamma of quarter s: the 8 values at k = 32h + 8s of the wavefront's private copy
        const uint32_t g_rd = lds0 + (uint32_t)(A_TILE_BYTES + wave * 256 + h * 64);
        // LDS destinations of this wavefront's loads within a stage
        const uint32_t lds_a = (uint32_t)(wave * TM * 1024);
        const uint32_t lds_g = (uint32_t)(A_TILE_BYTES + wave * 256);
        // the wavefront's weights of the next superstep; a lane's piece for K step x: piece 2 x + h of row l32
        const uint32_t lds_w = (uint32_t)(T::W_LDS_OFFSET + wave * TN * 4096);
        uint32_t w_rd[4];
#pragma unroll
        for (int x = 0; x < 4; ++x)
            w_rd[x] = lds0 + lds_w + (uint32_t)(l32 * 128 + (((2 * x + h) ^ ((l32 >> 1) & 7)) << 4));

        // (sync) the shared tiles this workgroup has parked a part of -- its first and its last segment -- and, in
        // thread 0, the tile's first sync word as the arrival found it
        __shared__ uint32_t sync_note[2];
        int pend_tile[2] = {-1, -1};
        uint32_t pend_old[2] = {0u, 0u};

        for (long long u = u_begin; u < u_end;)
        {
            // ---- this segment: tile and range of supersteps ----------------------------------------------------
            const int tile = (int)(u / SS);
            const int ss_begin = (int)(u - (long long)tile * SS);
            const int ss_end = (int)min((long long)SS, ss_begin + (u_end - u));
            const int NSS = ss_end - ss_begin;
            const bool whole = NSS == SS;
            const bool first_of_mine = u == u_begin;
            u += NSS;
            int tm, tn;
            {
                // four tile rows advance together along N
                constexpr int GM = 4;
                const int per_group = GM * p.tiles_n;
                const int g = tile / per_group;
                const int first_m = g * GM;
                const int gm = min(GM, p.tiles_m - first_m);
                const int r = tile - g * per_group;
                tm = first_m + r % gm;
                tn = r / gm;
            }
            const int m0 = tm * BM, n0 = tn * BN_OUT;
            const int k_begin = ss_begin * 256;
            const int KT = 4 * NSS;                             // K steps of this segment (the last two may lie past K)
            const int kt_max = min(KT, (K - k_begin) >> 6) - 1; // last K step inside K

            // ---- activations: direct-load map ------------------------------------------------------------------
            // chunk c fills LDS rows c*8 .. +7; lane l lands at (row = c*8 + l/8, slot = l%8) and therefore
            // fetches piece  slot ^ ((row >> 1) & 7)  of that row.  Wavefront w fetches chunks w*TM .. +TM-1.
            // (byte offsets from the operand's base: the matrices are below 4 GiB, checked by the launcher)
            uint32_t a_off[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i)
            {
                const int row = (wave * TM + i) * 8 + (lane >> 3);
                const int piece = (lane & 7) ^ ((row >> 1) & 7);
                a_off[i] = (uint32_t)(((size_t)min(m0 + row, p.M - 1) * K + k_begin + piece * 8) * 2);
            }
            const uint8_t* a_bytes = reinterpret_cast<const uint8_t*>(p.A);
            const uint8_t* g_bytes = reinterpret_cast<const uint8_t*>(p.gamma) + (size_t)k_begin * 2;
            const uint32_t g_off = (uint32_t)(lane & 31) * 4u;
            // scalar base of K step kt (clamped to the last inside K: past it a valid tile goes to a free stage, or is
            // multiplied by weights of zero)
            auto a_base_of = [&](int kt) { return scalar_base(a_bytes + (size_t)min(kt, kt_max) * (BK * 2)); };
            auto g_base_of = [&](int kt) { return scalar_base(g_bytes + (size_t)min(kt, kt_max) * (BK * 2)); };
            // activation load i of a K step -> stage
            auto load_a = [&](auto i_c, const uint8_t* a_base, uint32_t stage_off) {
                constexpr int i = decltype(i_c)::value;
                __builtin_amdgcn_global_load_lds((global_ptr)(a_base + here(a_off[i])), (lds_ptr)(smem + stage_off + lds_a + i * 1024), 16, 0, 0);
            };
            auto load_gamma = [&](const uint8_t* g_base, uint32_t stage_off) {
                __builtin_amdgcn_global_load_lds((global_ptr)(g_base + here(g_off)), (lds_ptr)(smem + stage_off + lds_g), 4, 0, 0);
            };

            // ---- weights and scales ----------------------------------------------------------------------------------
            // lane (l32, h) owns weight row l32 of each of the wavefront's column tiles; of K step t of a
            // superstep it owns k = 64 t + 32 h .. + 31: the 16 bytes at 32 t + 16 h of the superstep's 128.
            // Fetched that way -- 32 bytes of each of 32 rows per load -- the loads cost the memory pipeline four times
            // what whole 128-byte lines cost it (timed with the same bytes fetched as whole lines: M = 128, N = K = 8192
            // 32.0 -> 27.6 us).  So a superstep's 32 x 128 bytes per column tile go global -> LDS as whole lines, four
            // loads of 8 rows (lane i: row 8 c + i / 8, 16-byte piece (i % 8) ^ swizzle(row), as for the activations), into a
            // private area of the wavefront, one superstep ahead, and move into the registers with four ds_read_b128
            // when the superstep begins.
            // the row of the wavefront's column tile j that sits at place r (0 .. 31)
            auto weight_row = [&](int j, int r) {
                if (GATE) // column tiles 0 .. TN/2-1: gate rows, the others: the up rows that pair with them
                    return min((j >= TN / 2 ? p.up_row_offset + n0 + (j - TN / 2) * 32 : n0 + j * 32) + wave * (TN / 2) * 32 + r,
                               p.up_row_offset + p.N - 1);
                return min(n0 + wave * (TN * 32) + j * 32 + r, p.N - 1);
            };
            constexpr bool W_LDS = T::W_VIA_LDS;
            constexpr int WSETS = W_LDS ? 1 : 2; // register sets of weights: without the detour the next superstep's as well
            uint32_t w_off[TN][4], s_off[TN], z_off[TN]; // (straight into registers: w_off[j][0] only)
            // 64 in the lanes that fetch a piece of the second 64 bytes (K not a multiple of 256: they repeat the first
            // 64 in the last superstep), for loads 0 and 2 (the swizzle of rows 8 c + i / 8 flips it for loads 1 and 3)
            const uint32_t w_second_half = (lane & 4) ? 64u : 0u;
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                {
                    const int r = c * 8 + (lane >> 3);
                    const int piece = (lane & 7) ^ ((r >> 1) & 7);
                    w_off[j][c] = (uint32_t)((size_t)weight_row(j, r) * (K >> 1) + (k_begin >> 1) + piece * 16);
                }
                const int gn = weight_row(j, l32);
                if constexpr (!W_LDS)
                    w_off[j][0] = (uint32_t)((size_t)gn * (K >> 1) + (k_begin >> 1) + h * 16);
                if constexpr (QZ)
                {
                    // the scales of the row's groups of this superstep; their zero points, or (no tensor) the scales again
                    s_off[j] = (uint32_t)(((size_t)gn * G + (size_t)(256 >> GSH) * ss_begin) * 2);
                    z_off[j] = p.zps ? (uint32_t)((size_t)gn * (G >> 1) + (size_t)(128 >> GSH) * ss_begin) : s_off[j];
                }
                else
                    s_off[j] = (uint32_t)(((size_t)gn * G + 2 * ss_begin) * 2);
            }
            const uint8_t* s_bytes = reinterpret_cast<const uint8_t*>(p.S);
            // the weights of the superstep at work (set 0; straight into registers: and of the next one, set 1):
            // [set][column tile][K step of the superstep]
            uintx4 wbuf[WSETS][TN][4];
            uint32_t sraw[2][TN][SW]; // the group scales of the superstep, as loaded
            half2_t sc[2][TN][NSC];   // ... as (s, s); zero for a group past K
            uint32_t zraw[2][TN];     // QZ: the zero points of the superstep, as loaded
            half2_t dq[2][TN][NSC];   // QZ: (-(1024 + z), -(64 + z)) of the same groups
            // Scalar bases of superstep s of the segment (clamped to the last): weights of K steps 0 .. 1 and 2 .. 3,
            // first and second scale.  K not a multiple of 256: the last superstep has one group; its second half
            // repeats the first (and is multiplied by a scale of zero).
            struct WBase
            {
                const uint8_t *w, *s_lo, *s_hi;
                uint32_t repeat; // 64: the second 64 bytes of the superstep do not exist
            };
            auto w_base_of = [&](int s) {
                s = min(s, NSS - 1);
                WBase b;
                if constexpr (QZ)
                {
                    // (K is a multiple of 256)  s_lo: the scales; s_hi: the zero points, or the scales again
                    b.w = scalar_base(p.Wq + (size_t)s * 128);
                    b.repeat = 0u;
                    b.s_lo = scalar_base(s_bytes + (size_t)s * (512 >> GSH));
                    b.s_hi = p.zps ? scalar_base(p.zps + (size_t)s * (128 >> GSH)) : b.s_lo;
                    return b;
                }
                const bool second_valid = 2 * (ss_begin + s) + 1 < G;
                b.w = scalar_base(p.Wq + (size_t)s * 128);
                b.repeat = second_valid ? 0u : 64u;
                b.s_lo = scalar_base(s_bytes + (size_t)s * 4);
                b.s_hi = scalar_base(s_bytes + (size_t)s * 4 + (second_valid ? 2 : 0));
                return b;
            };
            // load x of column tile j.  0 .. 3: rows 8 x .. 8 x + 7 of its weights -> the wavefront's area in LDS;
            // 4 .. 5: scales -> register set
            auto load_w = [&](auto set_c, auto j_c, auto x_c, const WBase& b) {
                constexpr int set = decltype(set_c)::value, j = decltype(j_c)::value, x = decltype(x_c)::value;
                if constexpr (x < 4 && W_LDS)
                {
                    const uint32_t second = (x & 1) ? 64u - w_second_half : w_second_half;
                    __builtin_amdgcn_global_load_lds((global_ptr)(b.w + (here(w_off[j][x]) - (second & b.repeat))),
                                                     (lds_ptr)(smem + lds_w + j * 4096 + x * 1024), 16, 0, 0);
                }
                else if constexpr (x < 4) // the 16 bytes at 32 x + 16 h of the lane's own row
                    wbuf[set][j][x] = *(const uintx4 __attribute__((address_space(1)))*)(b.w + (x * 32 - (x >= 2 ? b.repeat : 0u)) + here(w_off[j][0]));
                else if constexpr (!QZ)
                {
                    // Loads 4 .. 6, the superstep's two scales of the lane's row.  A load costs by the lines it touches
                    // (32 rows here).  An even number of groups per row (K a multiple of 256): the two are one aligned
                    // word, load 4 brings it and loads 5 and 6 ask for the same two bytes in every lane (one line).
                    // An odd number: load 4 is the one that asks for one line, loads 5 and 6 bring a scale each.
                    // (One sequence of instructions for both: a branch around a load made the compiler drain every
                    // load in flight.)
                    const uint32_t mine = here(s_off[j]);
                    if constexpr (x == 4)
                        sraw[set][j][2] = *(const uint32_t __attribute__((address_space(1)))*)(b.s_lo + (g_even ? mine : 0u));
                    else if constexpr (x == 5)
                        sraw[set][j][0] = *(const uint16_t __attribute__((address_space(1)))*)(b.s_lo + (g_even ? 0u : mine));
                    else
                        sraw[set][j][1] = *(const uint16_t __attribute__((address_space(1)))*)((g_even ? b.s_lo : b.s_hi) + (g_even ? 0u : mine));
                }
                else if constexpr (x == 4)
                {
                    if constexpr (QG == 5)
                    {
                        const uintx4 v = *(const uintx4 __attribute__((address_space(1)))*)(b.s_lo + here(s_off[j]));
                        sraw[set][j][0] = v.x, sraw[set][j][1] = v.y, sraw[set][j][2] = v.z, sraw[set][j][3] = v.w;
                    }
                    else if constexpr (QG == 6)
                    {
                        const uintx2 v = *(const uintx2 __attribute__((address_space(1)))*)(b.s_lo + here(s_off[j]));
                        sraw[set][j][0] = v.x, sraw[set][j][1] = v.y;
                    }
                    else
                        sraw[set][j][0] = *(const uint32_t __attribute__((address_space(1)))*)(b.s_lo + here(s_off[j]));
                }
                else
                {
                    if constexpr (QG == 5)
                        zraw[set][j] = *(const uint32_t __attribute__((address_space(1)))*)(b.s_hi + here(z_off[j]));
                    else if constexpr (QG == 6)
                        zraw[set][j] = *(const uint16_t __attribute__((address_space(1)))*)(b.s_hi + here(z_off[j]));
                    else
                        zraw[set][j] = *(const uint8_t __attribute__((address_space(1)))*)(b.s_hi + here(z_off[j]));
                }
            };
            // QZ: a lane's group in K step t of a superstep is 2 t + h (groups of 32), t (64), t / 2 (128)
            const uint32_t h_sel = h ? 0x03020302u : 0x01000100u; // the half-word of a pair of scales that belongs to h
            const uint32_t z_and = p.zps ? 15u : 0u, z_or = p.zps ? 0u : (uint32_t)p.zp;
            // (s, s) of both groups of superstep s (as clamped by w_base_of)
            auto prepare_scales = [&](auto set_c, int s) {
                constexpr int set = decltype(set_c)::value;
                if constexpr (QZ)
                {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int i = 0; i < NSC; ++i)
                        {
                            uint32_t sv, z;
                            if constexpr (QG == 5)
                            {
                                sv = __builtin_amdgcn_perm(sraw[set][j][i], sraw[set][j][i], h_sel);
                                z = zraw[set][j] >> (uint32_t)(8 * i + 4 * h);
                            }
                            else
                            {
                                sv = __builtin_amdgcn_perm(sraw[set][j][i >> 1], sraw[set][j][i >> 1], (i & 1) ? 0x03020302u : 0x01000100u);
                                z = zraw[set][j] >> (uint32_t)(4 * i);
                            }
                            z = (z & z_and) | z_or;
                            sc[set][j][i] = as_half2(sv);
                            dq[set][j][i] = as_half2((z | (z << 20)) | 0xD400E400u);
                        }
                    return;
                }
                s = min(s, NSS - 1);
                const bool second_valid = 2 * (ss_begin + s) + 1 < G;
#pragma unroll
                for (int j = 0; j < TN; ++j)
                {
                    const uint32_t first = g_even ? sraw[set][j][2] : sraw[set][j][0];
                    const uint32_t second = g_even ? sraw[set][j][2] : sraw[set][j][1];
                    sc[set][j][0] = as_half2(__builtin_amdgcn_perm(first, first, 0x01000100u));
                    sc[set][j][1] = as_half2(second_valid ? __builtin_amdgcn_perm(second, second, g_even ? 0x03020302u : 0x01000100u) : 0u);
                }
            };

            floatx16 acc[TM][TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        acc[i][j][e] = 0.f;

            half8_t af[2][TM];     // activation fragments: two sets, used by alternating quarters
            uint32_t bw[2][TN][4]; // unpacked weight fragments, likewise
            uintx4 gm[4];          // RMS: gamma of the four quarters of a K step
            // Fragment reads the compiler does not track (it would wait for every LDS read in flight ahead of the first
            // use of any): valid after the wait of the region that uses them.  LDS operations complete in order.
            auto read_frag = [&](auto set_c, auto f_c, uint32_t addr) {
                lds_read_b128_nowait<decltype(f_c)::value * 4096>(af[decltype(set_c)::value][decltype(f_c)::value], addr);
            };
            // one half2 of the unpacked operand: weights 2e, 2e+1 of word `w` -> (q - zp) * scale (* gamma)
            // (QZ: `add` is the group's pair -(1024 + z), -(64 + z))
            auto unpack_piece_q = [&](auto set_c, auto j_c, auto e_c, uint32_t w, half2_t scale, half2_t add) {
                constexpr int set = decltype(set_c)::value, j = decltype(j_c)::value, e = decltype(e_c)::value;
                const uint32_t x = __builtin_amdgcn_perm(w, w, SEL[e]);
                const half2_t y = as_half2((x & MASK) | MAGIC);
                bw[set][j][e] = as_u32((y + add) * scale);
            };
            auto unpack_piece = [&](auto set_c, auto j_c, auto e_c, uint32_t w, half2_t scale, const uintx4& gam) {
                constexpr int set = decltype(set_c)::value, j = decltype(j_c)::value, e = decltype(e_c)::value;
                const uint32_t x = __builtin_amdgcn_perm(w, w, SEL[e]); // bytes (b_e, 0, b_e, 0)
                const half2_t y = as_half2((x & MASK) | MAGIC);         // (1024 + q_2e, 64 + q_2e+1)
                half2_t z = (y + dq_add) * scale;                       // (q - zp) * scale: one rounding
                if (RMS)
                    z = z * as_half2(e == 0 ? gam.x : e == 1 ? gam.y : e == 2 ? gam.z : gam.w);
                bw[set][j][e] = as_u32(z);
            };

            // ---- one K step --------------------------------------------------------------------------------------
            // Quarter q multiplies the fragments of k16 block q (operand set q & 1) while the other set is filled for
            // the next quarter.  Region r of a quarter: wait for its FPR fragments, ask for those of the next quarter,
            // FPR x TN MFMAs, a share of the next quarter's unpacking; wavefront r's loads of the quarter.
            //   t: K step within the superstep; s: superstep within the segment;
            //   prev_off / stage_off / next_off: LDS offsets of the stages of steps kt-1, kt, kt+1
            auto k_step = [&](auto t_c, int s, uint32_t prev_off, uint32_t stage_off, uint32_t next_off) {
                constexpr int T_ = decltype(t_c)::value;
                const int kt = 4 * s + T_;
                // loads of this step: positions 1 .. 3 of the activations of step kt+2 (-> the stage of step kt-1),
                // position 0 of step kt+3 (-> this step's stage), weights of superstep s+1
                const uint8_t* a_late = a_base_of(kt + 2);
                const uint8_t* a_next = a_base_of(kt + 3);
                const uint8_t* g_next = RMS ? g_base_of(kt + 3) : nullptr;
                const WBase w_next = w_base_of(s + 1);
                unroll_for<0, 4>([&](auto q_c) {
                    constexpr int Q = decltype(q_c)::value;
                    constexpr int SET = Q & 1, OTHER = SET ^ 1;
                    using OTHER_C = std::integral_constant<int, OTHER>;
                    if constexpr (Q == 3)
                    {
                        // every fragment of this step is in registers; step kt+1 has landed for this wavefront once only
                        // what it issued behind its loads is outstanding
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        __builtin_amdgcn_s_waitcnt(vmcnt_imm(SCH::later(T_)));
                        workgroup_barrier();
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr (T_ == 3)
                        {
                            prepare_scales(std::integral_constant<int, 1>{}, s + 1);
                            // the next superstep's weights have landed in the wavefront's area (the wait above), this
                            // superstep's are used up: LDS -> registers, waited for ahead of the first unpacking below
                            if constexpr (W_LDS)
                                unroll_for<0, TN>([&](auto j_c) {
                                    unroll_for<0, 4>([&](auto x_c) {
                                        lds_read_b128_nowait<decltype(j_c)::value * 4096>(wbuf[0][decltype(j_c)::value][decltype(x_c)::value],
                                                                                          w_rd[decltype(x_c)::value]);
                                    });
                                });
                        }
                    }
                    unroll_for<0, NREG>([&](auto r_c) {
                        constexpr int R = decltype(r_c)::value;
                        // the fragments of this region's MFMAs: behind the last of them, the reads of the regions after
                        // this one a quarter ago and of the regions before this one in this quarter
                        if constexpr (Q == 3)
                        {
                            unroll_for<0, FPR>([&](auto f_c) { lds_wait_also(af[SET][R * FPR + decltype(f_c)::value]); });
                        }
                        else
                        {
                            constexpr int DENSE = 2 * R < NREG ? 2 * R : NREG;
                            constexpr int BEHIND = (NREG - 1 - R) * FPR + (Q == 2 ? DENSE : R) * FPR;
                            lds_wait<BEHIND>(af[SET][R * FPR + FPR - 1]);
                            unroll_for<0, FPR - 1>([&](auto f_c) { lds_wait_also(af[SET][R * FPR + decltype(f_c)::value]); });
                        }
                        // RMS: gamma of the next K step (landed with its stage), all four quarters: quarters 1 .. 3 of
                        // this step's have been used up by the unpacking in quarters 0 .. 2, quarter 0's in the step before
                        if constexpr (RMS && Q == 3 && R == 0)
                            unroll_for<0, 4>([&](auto g_c) { lds_read_b128_nowait<decltype(g_c)::value * 16>(gm[decltype(g_c)::value], g_rd + next_off); });
                        // fragments of the next quarter (quarter 3's: two regions' worth per region, so that they have
                        // arrived at the barrier)
                        if constexpr (Q == 0 || Q == 1)
                            unroll_for<0, FPR>([&](auto f_c) {
                                read_frag(OTHER_C{}, std::integral_constant<int, R * FPR + decltype(f_c)::value>{}, a_rd[Q + 1] + stage_off);
                            });
                        else if constexpr (Q == 2)
                            unroll_for<0, 2 * FPR>([&](auto f_c) {
                                constexpr int F = 2 * R * FPR + decltype(f_c)::value;
                                if constexpr (F < TM)
                                    read_frag(OTHER_C{}, std::integral_constant<int, F>{}, a_rd[3] + stage_off);
                            });
                        else
                            unroll_for<0, FPR>([&](auto f_c) {
                                read_frag(OTHER_C{}, std::integral_constant<int, R * FPR + decltype(f_c)::value>{}, a_rd[0] + next_off);
                            });
                        // the MFMAs: the weight fragment is the first operand: D[n][m], lane (m = l32, h) holds four
                        // consecutive output columns per group of four elements, which is what the row-wise epilogue wants
#pragma unroll
                        for (int f = 0; f < FPR; ++f)
#pragma unroll
                            for (int j = 0; j < TN; ++j)
                                acc[R * FPR + f][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                                    __builtin_bit_cast(half8_t, uintx4{bw[SET][j][0], bw[SET][j][1], bw[SET][j][2], bw[SET][j][3]}),
                                    af[SET][R * FPR + f], acc[R * FPR + f][j], 0, 0, 0);
                        // this region's share of the unpacking for the next quarter: pieces (j, e).  (RMS, quarter 3: the
                        // gamma values have just been asked for: the unpacking starts one region later.)
                        constexpr int PIECES = 4 * TN;
                        constexpr bool SHIFTED = RMS && Q == 3 && NREG > 1;
                        constexpr int NR1 = NREG > 1 ? NREG - 1 : 1;
                        constexpr int P0 = SHIFTED ? (R == 0 ? 0 : (R - 1) * PIECES / NR1) : R * PIECES / NREG;
                        constexpr int P1 = SHIFTED ? (R == 0 ? 0 : R * PIECES / NR1) : (R + 1) * PIECES / NREG;
                        if constexpr (RMS && Q == 3 && (NREG > 1 ? R == 1 : R == 0))
                        {
                            // behind the gamma reads: the fragment reads of the regions so far
                            lds_wait<(NREG > 1 ? 2 * FPR : FPR)>(gm[0]);
                            lds_wait_also(gm[1]);
                            lds_wait_also(gm[2]);
                            lds_wait_also(gm[3]);
                        }
                        if constexpr (W_LDS && Q == 3 && T_ == 3 && (SHIFTED ? R == 1 : R == 0))
                        {
                            // the weights read back at the top of this quarter: behind them this region's fragment reads
                            // (RMS: the wait above was stricter)
                            if constexpr (!RMS)
                                lds_wait<FPR>(wbuf[0][0][0]);
                            unroll_for<0, 4 * TN>([&](auto i_c) { lds_wait_also(wbuf[0][decltype(i_c)::value / 4][decltype(i_c)::value % 4]); });
                        }
                        unroll_for<P0, P1>([&](auto pc_c) {
                            constexpr int pc = decltype(pc_c)::value;
                            constexpr int j = pc / 4, e = pc % 4;
                            // word Q+1 of this step, or word 0 of the next step
                            constexpr int NT = Q == 3 ? (T_ + 1) & 3 : T_;
                            constexpr int NSET = (Q == 3 && T_ == 3) ? 1 : 0; // (the scales; the weights are in place by then)
                            constexpr int NQ = (Q + 1) & 3;
                            const uintx4& wq = wbuf[W_LDS ? 0 : NSET][j][NT];
                            const uint32_t w = NQ == 0 ? wq.x : NQ == 1 ? wq.y : NQ == 2 ? wq.z : wq.w;
                            if constexpr (QZ)
                            {
                                constexpr int SI = QG != 7 ? NT : NT >> 1; // the group of K step NT
                                unpack_piece_q(OTHER_C{}, std::integral_constant<int, j>{}, std::integral_constant<int, e>{}, w,
                                               sc[NSET][j][SI], dq[NSET][j][SI]);
                            }
                            else
                                unpack_piece(OTHER_C{}, std::integral_constant<int, j>{}, std::integral_constant<int, e>{}, w,
                                             sc[NSET][j][NT >> 1], gm[NQ]);
                        });
                        // this quarter's loads, spread over its regions
                        constexpr int N_W = Q < 3 ? SCH::w_begin(T_, Q + 1) - SCH::w_begin(T_, Q) : 0;
                        constexpr int N_A = SCH::a_loads_at(Q == 3 ? 0 : Q + 1) - ((RMS && Q == 3) ? 1 : 0);
                        constexpr int N_L = N_W + N_A + ((RMS && Q == 3) ? 1 : 0);
                        unroll_for<R * N_L / NREG, (R + 1) * N_L / NREG>([&](auto l_c) {
                            constexpr int L = decltype(l_c)::value;
                            if constexpr (L < N_W)
                            {
                                constexpr int X = SCH::w_begin(T_, Q) + L;
                                load_w(std::integral_constant<int, 1>{}, std::integral_constant<int, SCH::w_tile(T_, X)>{},
                                       std::integral_constant<int, SCH::w_which(X)>{}, w_next);
                            }
                            else if constexpr (L < N_W + N_A)
                            {
                                // the (L - N_W)-th activation load of this position
                                constexpr int POS = Q == 3 ? 0 : Q + 1;
                                constexpr int FIRST = (POS * TM + 3) / 4; // smallest i with a_pos(i) == POS
                                static_assert(SCH::a_pos(FIRST + L - N_W) == POS, "activation loads of a position are consecutive");
                                load_a(std::integral_constant<int, FIRST + L - N_W>{}, Q == 3 ? a_next : a_late, Q == 3 ? stage_off : prev_off);
                            }
                            else
                                load_gamma(g_next, stage_off);
                        });
                        asm volatile("" ::: "memory");
                        __builtin_amdgcn_sched_barrier(0);
                    });
                });
                // the accumulators stay in the accumulation registers
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        asm volatile("" : "+a"(acc[i][j]));
            };

            // ---- K loop ---------------------------------------------------------------------------------------
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            using I3 = std::integral_constant<int, 3>;
            {
                // steps 0 and 1 and superstep 0 in full, of step 2 what quarter 3 of a step before the first would
                // have asked for
                const WBase w0 = w_base_of(0);
                unroll_for<0, TM>([&](auto i_c) { load_a(i_c, a_base_of(0), 0u); });
                unroll_for<0, TN>([&](auto j_c) { unroll_for<0, NW>([&](auto x_c) { load_w(I0{}, j_c, x_c, w0); }); });
                if constexpr (RMS)
                    load_gamma(g_base_of(0), 0u);
                unroll_for<0, TM>([&](auto i_c) { load_a(i_c, a_base_of(1), (uint32_t)STAGE_BYTES); });
                if constexpr (RMS)
                    load_gamma(g_base_of(1), (uint32_t)STAGE_BYTES);
                unroll_for<0, TM>([&](auto i_c) {
                    if constexpr (SCH::a_pos(decltype(i_c)::value) == 0)
                        load_a(i_c, a_base_of(2), (uint32_t)(2 * STAGE_BYTES));
                });
                if constexpr (RMS)
                    load_gamma(g_base_of(2), (uint32_t)(2 * STAGE_BYTES));
            }
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(SCH::a_loads_total() + SCH::a_loads_at(0))); // step 0 and superstep 0 have landed
            workgroup_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (first_of_mine)
                NNF_SK_STAMP(1); // the first operands have arrived
            else if (u >= u_end)
                NNF_SK_STAMP(12); // ... and those of the last segment, when it is not the first
            prepare_scales(I0{}, 0);
            // superstep 0's weights: LDS -> registers
            if constexpr (W_LDS)
                unroll_for<0, TN>([&](auto j_c) {
                    unroll_for<0, 4>([&](auto x_c) {
                        lds_read_b128_nowait<decltype(j_c)::value * 4096>(wbuf[0][decltype(j_c)::value][decltype(x_c)::value], w_rd[decltype(x_c)::value]);
                    });
                });
            if constexpr (RMS)
                unroll_for<0, 4>([&](auto g_c) { lds_read_b128_nowait<decltype(g_c)::value * 16>(gm[decltype(g_c)::value], g_rd); });
            unroll_for<0, TM>([&](auto f_c) { read_frag(I0{}, f_c, a_rd[0]); });
            if constexpr (RMS)
            {
                lds_wait<(TM < 15 ? TM : 15)>(gm[0]);
                lds_wait_also(gm[1]);
                lds_wait_also(gm[2]);
                lds_wait_also(gm[3]);
            }
            else if constexpr (W_LDS)
                lds_wait<(TM < 15 ? TM : 15)>(wbuf[0][0][0]);
            if constexpr (W_LDS)
                unroll_for<0, 4 * TN>([&](auto i_c) { lds_wait_also(wbuf[0][decltype(i_c)::value / 4][decltype(i_c)::value % 4]); });
            unroll_for<0, 4 * TN>([&](auto pc_c) {
                constexpr int pc = decltype(pc_c)::value;
                if constexpr (QZ)
                    unpack_piece_q(I0{}, std::integral_constant<int, pc / 4>{}, std::integral_constant<int, pc % 4>{}, wbuf[0][pc / 4][0].x,
                                   sc[0][pc / 4][0], dq[0][pc / 4][0]);
                else
                    unpack_piece(I0{}, std::integral_constant<int, pc / 4>{}, std::integral_constant<int, pc % 4>{}, wbuf[0][pc / 4][0].x,
                                 sc[0][pc / 4][0], gm[0]);
            });
            __builtin_amdgcn_sched_barrier(0);
            // No LDS read other than the fragments of quarter 0 is in flight at the top of a K step.
            {
                constexpr uint32_t RING = (uint32_t)(STAGES * STAGE_BYTES);
                auto next_of = [](uint32_t o) { return o + STAGE_BYTES == RING ? 0u : o + (uint32_t)STAGE_BYTES; };
                uint32_t pv = RING - (uint32_t)STAGE_BYTES, st = 0;
                // one loop body: the superstep works on register set 0 and fills set 1, which moves to set 0 at its end
                // (a few dozen register moves per 256 MFMAs; two bodies that swap the roles of the sets instead measured the
                // same at every M, and spilled registers under the 256 x 256 tile)
                for (int s = 0; s < NSS; ++s)
                {
                    k_step(I0{}, s, pv, st, next_of(st));
                    pv = st, st = next_of(st);
                    k_step(I1{}, s, pv, st, next_of(st));
                    pv = st, st = next_of(st);
                    k_step(I2{}, s, pv, st, next_of(st));
                    pv = st, st = next_of(st);
                    k_step(I3{}, s, pv, st, next_of(st));
                    pv = st, st = next_of(st);
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                    {
                        if constexpr (!W_LDS)
                        {
#pragma unroll
                            for (int x = 0; x < 4; ++x)
                                wbuf[0][j][x] = wbuf[WSETS - 1][j][x];
                        }
                        if constexpr (QZ)
                        {
#pragma unroll
                            for (int i = 0; i < NSC; ++i)
                                sc[0][j][i] = sc[1][j][i], dq[0][j][i] = dq[1][j][i];
                        }
                        else
                        {
                            sc[0][j][0] = sc[1][j][0];
                            sc[0][j][1] = sc[1][j][1];
                        }
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the fragments read ahead for a step that does not exist
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));          // nothing may land in LDS or in registers any more ...
            __syncthreads();                                   // ... from any wavefront: the ring is free
            if (u >= u_end)
                NNF_SK_STAMP(2); // the K loop of the last segment is over
            else if (first_of_mine)
                NNF_SK_STAMP(10); // ... of the first segment, when it is not the last

            // ---- a tile shared with other workgroups: park the sums in register order (element block q of MFMA tile
            // (i, j) of all 256 threads is one contiguous 4 KiB); w4a16_gemm_sk_fixup_kernel adds the parts and finishes
            if (!whole)
            {
                const size_t first_float = ((size_t)v + (first_of_mine ? 0 : (size_t)grid)) * T::SLOT_FLOATS + (size_t)tid * 4;
                float* mine = p.partial + first_float;
                const bool same_launch = p.sync != nullptr;
                const buffer_t parked = parked_buffer(p.partial, p.partial_bytes);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                        {
                            const size_t at = (size_t)(((i * TN + j) * 4 + q) * THREADS * 4);
                            const floatx4 part = floatx4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                            if (same_launch)
                                store_device_scope(parked, (uint32_t)((first_float + at) * sizeof(float)), part);
                            else
                                *reinterpret_cast<floatx4*>(mine + at) = part;
                            __builtin_amdgcn_sched_barrier(0); // (one quarter of a tile at a time: few registers)
                        }
                if (same_launch)
                {
                    // every wavefront's part has arrived where every CU sees it before thread 0 counts the workgroup in
                    wait_vector_memory();
                    __syncthreads();
                    if (u >= u_end)
                        NNF_SK_STAMP(3); // its part is parked
                    uint32_t old = 0u;
                    if (tid == 0)
                        old = atomicAdd(p.sync + 2 * (size_t)tile, 1u);
                    if (u >= u_end)
                        NNF_SK_STAMP(4 + (old & 0u)); // ... and counted in
                    else if (first_of_mine)
                        NNF_SK_STAMP(11 + (old & 0u)); // (the first segment's part, when it is not the last)
                    if (first_of_mine)
                        pend_tile[0] = tile, pend_old[0] = old;
                    else
                        pend_tile[1] = tile, pend_old[1] = old;
                }
            }
            else
            {
                // ---- epilogue: two blocks of 32 rows at a time ------------------------------------------------------
                constexpr int ROUND_TM = TM >= 2 ? 2 : 1;
                ensure_rstd(m0, m0 + BM);
#pragma unroll
                for (int r = 0; r < TM / ROUND_TM; ++r)
                {
                    floatx16 c[ROUND_TM][TN];
#pragma unroll
                    for (int ii = 0; ii < ROUND_TM; ++ii)
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            c[ii][j] = acc[r * ROUND_TM + ii][j];
                    sk_finish_round<TM, TN, GATE, BIAS, RESID, RMS>(p, c, r, m0, n0, smem + wave * sk_region_bytes<TM, TN, GATE>(), wave, lane);
                    __builtin_amdgcn_sched_barrier(0); // (one round at a time: few registers)
                }
            }
            if (u < u_end)
                __syncthreads(); // the staging regions are read before the next segment's tiles land in them
        }

        // ---- (sync) shared tiles: once every workgroup that holds a part has arrived, each of them adds up and
        // finishes its share of the tile's 32-row blocks (block i belongs to the (i mod n)-th of the n workgroups).
        // Every workgroup has counted itself in at all its tiles before it waits here, so the waits cannot form a
        // cycle; they are bounded all the same (workgroups of a grid that is not resident as a whole): a workgroup
        // whose wait runs out marks its blocks for the last arriver, who never waits.
        if (p.sync && (pend_tile[0] >= 0 || pend_tile[1] >= 0))
        {
            __syncthreads(); // the epilogue's staging regions are free
            uint8_t* stage = smem + wave * sk_region_bytes<1, TN, GATE>();
            SkSharedTile shared[2];
            uint32_t blocks[2] = {0u, 0u};
#pragma unroll
            for (int slot = 0; slot < 2; ++slot)
            {
                const int tile = pend_tile[slot];
                const long long t0 = (long long)max(tile, 0) * SS;
                shared[slot].tile = tile;
                shared[slot].v_first = owner_of_unit(t0, p.units, grid);
                shared[slot].n_seg = owner_of_unit(t0 + SS - 1, p.units, grid) - shared[slot].v_first + 1;
                shared[slot].first_is_second_slot = first_unit_of(shared[slot].v_first, p.units, grid) < t0;
                if (tile >= 0 && tid == 0)
                {
                    uint32_t own = 0u;
                    for (int i = v - shared[slot].v_first; i < TM; i += shared[slot].n_seg)
                        own |= 1u << i;
                    sync_note[slot] = sk_blocks_to_finish(p.sync + 2 * (size_t)tile, pend_old[slot], shared[slot].n_seg, own, p.spin_limit);
                }
            }
            __syncthreads();
            blocks[0] = pend_tile[0] >= 0 ? sync_note[0] : 0u;
            blocks[1] = pend_tile[1] >= 0 ? sync_note[1] : 0u;
            NNF_SK_STAMP(5); // the waits for the tiles' other workgroups are over
            if constexpr (RMS)
            {
#pragma unroll
                for (int slot = 0; slot < 2; ++slot)
                    if (blocks[slot]) // (uniform)
                    {
                        // the tile's rows (tiles are numbered as in the K loop: four tile rows advance together along N)
                        const int per_group = 4 * p.tiles_n;
                        const int g = shared[slot].tile / per_group;
                        const int gm = min(4, p.tiles_m - g * 4);
                        const int tm = g * 4 + (shared[slot].tile - g * per_group) % gm;
                        ensure_rstd(tm * BM, tm * BM + BM);
                    }
            }
            // (every part was complete at device scope before its workgroup counted itself in, the counts were read at
            // device scope, and so are the parts)
            // The blocks to finish, those of the first tile in bits 0 .. 7, of the second in bits 8 .. 15, one after the
            // other; where the registers allow it the parts of the next block are asked for ahead of this block's sums.
            constexpr bool AHEAD = sk_loads_ahead<TM, TN>();
            uint32_t todo = blocks[0] | (blocks[1] << 8);
            // (selected field by field: an array indexed at run time would live in private memory)
            auto tile_of = [&](int task) {
                const bool second = task >= 8;
                SkSharedTile t;
                t.tile = second ? shared[1].tile : shared[0].tile;
                t.v_first = second ? shared[1].v_first : shared[0].v_first;
                t.n_seg = second ? shared[1].n_seg : shared[0].n_seg;
                t.first_is_second_slot = second ? shared[1].first_is_second_slot : shared[0].first_is_second_slot;
                return t;
            };
            if constexpr (AHEAD)
            {
                SkPartsInFlight<TM, TN, true> x0, x1;
                int cur = todo ? __builtin_ctz(todo) : -1;
                if (cur >= 0)
                    sk_request_parts<TM, TN, true>(x0, p, grid, tile_of(cur), cur & 7, 0, tid);
                while (cur >= 0)
                {
                    todo &= todo - 1;
                    int nxt = todo ? __builtin_ctz(todo) : -1;
                    if (nxt >= 0)
                        sk_request_parts<TM, TN, true>(x1, p, grid, tile_of(nxt), nxt & 7, 0, tid);
                    sk_finish_block<TM, TN, GATE, BIAS, RESID, RMS, true>(x0, p, grid, tile_of(cur), cur & 7, stage, wave, lane);
                    if (nxt < 0)
                        break;
                    todo &= todo - 1;
                    cur = todo ? __builtin_ctz(todo) : -1;
                    if (cur >= 0)
                        sk_request_parts<TM, TN, true>(x0, p, grid, tile_of(cur), cur & 7, 0, tid);
                    sk_finish_block<TM, TN, GATE, BIAS, RESID, RMS, true>(x1, p, grid, tile_of(nxt), nxt & 7, stage, wave, lane);
                }
            }
            else
            {
                SkPartsInFlight<TM, TN, true> x;
                while (todo)
                {
                    const int cur = __builtin_ctz(todo);
                    todo &= todo - 1;
                    sk_request_parts<TM, TN, true>(x, p, grid, tile_of(cur), cur & 7, 0, tid);
                    sk_finish_block<TM, TN, GATE, BIAS, RESID, RMS, true>(x, p, grid, tile_of(cur), cur & 7, stage, wave, lane);
                }
            }
            __syncthreads(); // every wavefront's strips are finished
            NNF_SK_STAMP(6); // this workgroup's share of its tiles is finished
            if (tid == 0)
            {
#pragma unroll
                for (int slot = 0; slot < 2; ++slot)
                    if (blocks[slot])
                    {
                        uint32_t* state = p.sync + 2 * (size_t)pend_tile[slot];
                        const uint32_t n = (uint32_t)__builtin_popcount(blocks[slot]);
                        if (atomicAdd(state + 1, n) + n == (uint32_t)TM)
                        {
                            // nobody looks at this tile's words any more: leave them as the next launch wants them
                            atomicExch(state, 0u);
                            atomicExch(state + 1, 0u);
                        }
                    }
            }
        }
        if constexpr (RMS)
        {
            // (rstd_out) the last workgroup to end leaves the two words as the next launch wants them
            if (p.rstd_out && tid == 0 && atomicAdd(p.rstd_sync + 1, 1u) == (uint32_t)(grid - 1))
            {
                atomicExch(p.rstd_sync, 0u);
                atomicExch(p.rstd_sync + 1, 0u);
            }
        }
        NNF_SK_STAMP(9); // done
    }

    // launches w4a16_gemm_sk_kernel<...> on `grid` workgroups
    template <class Kernel>
    inline void launch_sk_kernel(Kernel kernel, int grid, size_t lds_bytes, hipStream_t stream, const SkGemmParams& p)
    {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(gemm_sk::THREADS), lds_bytes, stream, p.A, p.Wq, p.S, p.units, p.M, p.N, p.K,
                           p.tiles_n, p.supersteps, grid, p);
    }

    // Adds the parts of the tiles that several workgroups of w4a16_gemm_sk_kernel worked on, in K order (so the result
    // does not depend on timing), and runs the epilogue.  The strips of the GEMM's four wavefronts are independent of one
    // another here: one workgroup of a single wavefront per tile, block of 32 rows and strip (a few dozen tiles
    // then still spread over all CUs); one whose tile had a single owner has nothing to do.  `gemm_grid`: workgroups of
    // the GEMM launch.
    template <int TM, int TN, bool GATE, bool BIAS, bool RESID, bool RMS>
    __global__ __launch_bounds__(64) void w4a16_gemm_sk_fixup_kernel(SkGemmParams p, int gemm_grid)
    {
        using namespace gemm_sk;
        constexpr int ROUND_TM = 1, ROUNDS = TM; // (the epilogue routine of a tile one block high)
        __shared__ __attribute__((aligned(16))) uint8_t stage[ROUND_TM * 32 * (TN * 64 + 16)];
        const int lane = threadIdx.x;
        const int wave = (int)blockIdx.x % WAVES; // the strip: what wavefront `wave` of the GEMM's workgroup parked
        const int tile = (int)blockIdx.x / (WAVES * ROUNDS), r = ((int)blockIdx.x / WAVES) % ROUNDS;
        const int SS = p.supersteps;
        const long long t0 = (long long)tile * SS;
        const int v_first = owner_of_unit(t0, p.units, gemm_grid);
        const int n_seg = owner_of_unit(t0 + SS - 1, p.units, gemm_grid) - v_first + 1;
        if (n_seg == 1)
            return;
        // the first owner parked this tile in its second slot when its range began in an earlier tile
        const bool first_is_second_slot = first_unit_of(v_first, p.units, gemm_grid) < t0;
        SkSharedTile t;
        t.tile = tile, t.v_first = v_first, t.n_seg = n_seg, t.first_is_second_slot = first_is_second_slot;
        SkPartsInFlight<TM, TN, false> x;
        sk_request_parts<TM, TN, false>(x, p, gemm_grid, t, r, 0, wave * 64 + lane);
        sk_finish_block<TM, TN, GATE, BIAS, RESID, RMS, false>(x, p, gemm_grid, t, r, stage, wave, lane);
    }
} // namespace nnf
