// fp16 activations x 4- or 8-bit weights with the block parameters the specialised kernels do not take: groups of
// 32 / 64 / 128, one zero point per (row, group), 8-bit weights.
//
//   Y[M,N] = A[M,K] . ((Wq - zero point) * S)^T
//
// The reference's dequantize takes a scale and an offset per block of any shape
// (src/nnfusion/core/kernels/cpu/reference/kernels.cpp:601-623: integer subtract of the offset, cast, multiply by
// the scale); the kernels in w4a16_*.hip serve the one combination the benchmark uses (4 bits, groups of 128, a
// scalar zero point) as fast as the hardware allows, these serve every other one correctly and simply:
//   * wna16_gemv_kernel (M = 1 where K is not a multiple of 256; the others run on the row-streaming kernel of
//     w4a16_gemv_rows.hip, 4- and 8-bit weights alike): a wavefront per block of four weight rows; a lane turns 16
//     bytes of weights of each into the exact integers q - z in fp16, multiplies them with the activations
//     (v_dot2_f32_f16, fp32 sums) and applies the group's scale to the sum over its piece of the group;
//   * wna16_skinny_kernel (2 <= M <= 16): v_mfma_f32_16x16x32_f16, activations and weights fetched straight into the
//     operand registers, eight wavefronts share the K range of two tiles of 16 weight rows;
//   * wna16_tile_kernel (M > 16): 64 x 64, 128 x 128, 256 x 128 or 256 x 256 output tiles (the shape with the lowest
//     estimated time) on v_mfma_f32_32x32x16_f16, K steps of 64 through two LDS buffers, the operands of the step after
//     next on their way into registers and the next step's on their way into LDS while this step's MFMAs run.
// The MFMA kernels dequantise to fp16((q - z) * s) (what the specialised tile GEMM's unpacking produces as well).
#include "nnf_device.h"
#include "nnf_launch.h"

namespace nnf
{
    namespace
    {
        struct QuantArgs
        {
            const uint8_t* zps; // per-(row, group) zero points or null
            int group_shift;    // log2 of the group size (32, 64 or 128)
            int zp;             // scalar zero point (zps == null)
            int zp_stride;      // bytes per row of zps
        };

        template <int BITS>
        __device__ __forceinline__ int zero_point_of(const QuantArgs& qa, int n, int g)
        {
            if (!qa.zps)
                return qa.zp;
            if constexpr (BITS == 4)
            {
                const uint8_t b = qa.zps[(size_t)n * qa.zp_stride + (g >> 1)];
                return (g & 1) ? (b >> 4) : (b & 0xF);
            }
            else
                return qa.zps[(size_t)n * qa.zp_stride + g];
        }
    } // namespace

    // The exact integers (q - z) of eight weights as four fp16 pairs (|q - z| <= 255), by the offset trick of dequant8
    // (nnf_device.h): a byte or nibble placed in the mantissa of 1024.0 is 1024 + q, and subtracting 1024 + z is exact.
    // 4 bits: `w` holds the eight, pairs come out as (0,4) (1,5) (2,6) (3,7); 8 bits: `w` then `w_hi`, pairs in order.
    template <int BITS>
    struct ExactWeights
    {
        DequantConst c4;
        half2_t c8;
        __device__ __forceinline__ explicit ExactWeights(int z)
        {
            if constexpr (BITS == 4)
                c4 = make_dequant_const(z);
            else
            {
                const half_t c = (half_t)(-(1024.0f + (float)z));
                c8 = half2_t{c, c};
            }
        }
        __device__ __forceinline__ void operator()(uint32_t w, uint32_t w_hi, half2_t (&out)[4]) const
        {
            if constexpr (BITS == 4)
                dequant8(w, c4, out);
            else
            {
                // v_perm_b32(S0, S1, sel): selectors 0-3 pick bytes of S1, 4-7 of S0
                out[0] = as_half2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) + c8;
                out[1] = as_half2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) + c8;
                out[2] = as_half2(__builtin_amdgcn_perm(0x64646464u, w_hi, 0x04010400u)) + c8;
                out[3] = as_half2(__builtin_amdgcn_perm(0x64646464u, w_hi, 0x04030402u)) + c8;
            }
        }
    };

    // grid: any; each wavefront walks blocks of R consecutive rows (R x its number, + R x the number of wavefronts, ...);
    // a lane takes 16 bytes of each of the R rows per pass over K (32 or 16 weights, inside one group): the sum of
    // a x (q - z) over them (v_dot2_f32_f16 on exact operands) times the group's scale is added to the lane's fp32 sums.
    // The activations a lane meets are fetched once per pass for all R rows.  MB: upper bound of M.
    template <int BITS, int R, int MB>
    __global__ __launch_bounds__(256) void wna16_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                             const half_t* __restrict__ S, half_t* __restrict__ Y, int M, int N,
                                                             int K, QuantArgs qa)
    {
        constexpr int WPL = 128 / BITS; // weights per lane and pass
        const int lane = threadIdx.x & 63;
        const int wave = (int)blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = (int)gridDim.x * 4;
        const int G = K >> qa.group_shift;
        const size_t row_bytes = (size_t)K * BITS / 8;
        for (int n = wave * R; n < N; n += n_waves * R)
        {
            int row[R]; // (rows past the end of a ragged N are computed on the last row and dropped)
            float acc[MB][R];
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                row[r] = min(n + r, N - 1);
#pragma unroll
                for (int m = 0; m < MB; ++m)
                    acc[m][r] = 0.f;
            }
            for (int k = lane * WPL; k < K; k += 64 * WPL)
            {
                const int g = k >> qa.group_shift;
                uintx4 w[R];
                float sc[R];
                int z[R];
#pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    w[r] = *reinterpret_cast<const uintx4*>(Wq + (size_t)row[r] * row_bytes + (size_t)k * BITS / 8);
                    z[r] = zero_point_of<BITS>(qa, row[r], g);
                    sc[r] = (float)S[(size_t)row[r] * G + g];
                }
                float part[MB][R];
#pragma unroll
                for (int m = 0; m < MB; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        part[m][r] = 0.f;
#pragma unroll
                for (int p = 0; p < WPL / 8; ++p)
                {
                    half2_t v[R][4];
#pragma unroll
                    for (int r = 0; r < R; ++r)
                    {
                        const ExactWeights<BITS> exact(z[r]);
                        if constexpr (BITS == 4)
                            exact(w[r][p], 0u, v[r]);
                        else
                            exact(w[r][2 * p], w[r][2 * p + 1], v[r]);
                    }
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        if (m < M)
                        {
                            uintx4 a = *reinterpret_cast<const uintx4*>(A + (size_t)m * K + k + 8 * p);
                            if constexpr (BITS == 4)
                                a = permute_a8(a);
#pragma unroll
                            for (int i = 0; i < 4; ++i)
#pragma unroll
                                for (int r = 0; r < R; ++r)
                                    part[m][r] = dot2(as_half2(a[i]), v[r][i], part[m][r]);
                        }
                }
#pragma unroll
                for (int m = 0; m < MB; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        acc[m][r] = __builtin_fmaf(part[m][r], sc[r], acc[m][r]);
            }
#pragma unroll
            for (int m = 0; m < MB; ++m)
                if (m < M)
                {
#pragma unroll
                    for (int r = 0; r < R; ++r)
                    {
                        const float t = wave_sum(acc[m][r]);
                        if (lane == 0 && n + r < N)
                            Y[(size_t)m * N + n + r] = (half_t)t;
                    }
                }
        }
    }

    template <int BITS, int R, int MB>
    void launch_wna16_gemv(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                           const QuantArgs& qa, int num_cu)
    {
        // enough wavefronts to cover the blocks of rows once, at most eight workgroups of four per CU
        const int want = (N + 4 * R - 1) / (4 * R), cap = num_cu * 8;
        hipLaunchKernelGGL((wna16_gemv_kernel<BITS, R, MB>), dim3((unsigned)(want < cap ? want : cap)), dim3(256), 0, stream,
                           (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, M, N, K, qa);
    }

    // 2 <= M <= 16 on the matrix cores (v_mfma_f32_16x16x32_f16: activations as the 16-row operand, 16 weight rows as
    // the other).  A workgroup of eight wavefronts walks blocks of NT tiles of 16 weight rows; the wavefronts take the
    // chunks of K in turn (a chunk: 4 x 16 bytes of each weight row, 128 or 64 values of K): lane (row l % 16, quarter
    // l / 16) fetches 16 bytes of its row of every tile and the activations of the same K positions of row l % 16 (once
    // for the NT tiles) straight into the MFMA operand registers (the next chunk's while this one is computed),
    // dequantises to fp16((q - z) * s) (the exact integers by the offset trick, one rounding in the multiply) and issues
    // one MFMA per tile and eight values of K.  The eight partial 16 x 16 tiles of every tile meet in LDS.
    constexpr int SKINNY_WAVES = 8;
    template <int BITS, int NT>
    __global__ __launch_bounds__(SKINNY_WAVES * 64) void wna16_skinny_kernel(const half_t* __restrict__ A,
                                                                             const uint8_t* __restrict__ Wq,
                                                                             const half_t* __restrict__ S, half_t* __restrict__ Y,
                                                                             int M, int N, int K, QuantArgs qa)
    {
        constexpr int WPL = 128 / BITS;  // weights per lane, tile and chunk
        constexpr int PIECES = WPL / 8;  // MFMAs per tile and chunk
        constexpr int CHUNK = 4 * WPL;   // values of K per chunk
        __shared__ __attribute__((aligned(16))) floatx4 red[SKINNY_WAVES][NT][64];
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int col = lane & 15, kq = lane >> 4;
        const int G = K >> qa.group_shift;
        const size_t row_bytes = (size_t)K * BITS / 8;
        const int n_chunks = (K + CHUNK - 1) / CHUNK;
        const half_t* a_row = A + (size_t)min(col, M - 1) * K; // (rows past M repeat the last one and are dropped)
        struct Operands
        {
            uintx4 w[NT], a[PIECES];
            float s[NT];
            int z[NT];
        };
        for (int block = (int)blockIdx.x; block * (16 * NT) < N; block += (int)gridDim.x)
        {
            int n[NT]; // (rows past N repeat the last one and are dropped)
#pragma unroll
            for (int t = 0; t < NT; ++t)
                n[t] = min((block * NT + t) * 16 + col, N - 1);
            auto fetch = [&](int c, Operands& o) {
                // a lane past the end of K (the last chunk of a K that is not a multiple of it) repeats the row's last
                // piece with a scale of zero
                const int k_raw = c * CHUNK + kq * WPL;
                const int k = min(k_raw, K - WPL);
                const int g = k >> qa.group_shift;
#pragma unroll
                for (int t = 0; t < NT; ++t)
                {
                    o.w[t] = *reinterpret_cast<const uintx4*>(Wq + (size_t)n[t] * row_bytes + (size_t)k * BITS / 8);
                    o.z[t] = zero_point_of<BITS>(qa, n[t], g);
                    o.s[t] = k_raw < K ? (float)S[(size_t)n[t] * G + g] : 0.f;
                }
#pragma unroll
                for (int p = 0; p < PIECES; ++p)
                    o.a[p] = *reinterpret_cast<const uintx4*>(a_row + k + 8 * p);
            };
            floatx4 acc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
            Operands cur, nxt;
            if (wave < n_chunks)
                fetch(wave, cur);
            for (int c = wave; c < n_chunks; c += SKINNY_WAVES)
            {
                if (c + SKINNY_WAVES < n_chunks)
                    fetch(c + SKINNY_WAVES, nxt);
#pragma unroll
                for (int p = 0; p < PIECES; ++p)
                {
                    uintx4 a = cur.a[p];
                    if constexpr (BITS == 4)
                        a = permute_a8(a); // the pair order of the unpacked nibbles
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                    {
                        const ExactWeights<BITS> exact(cur.z[t]);
                        const half_t sh = (half_t)cur.s[t];
                        const half2_t s2 = half2_t{sh, sh};
                        half2_t v[4];
                        if constexpr (BITS == 4)
                            exact(cur.w[t][p], 0u, v);
                        else
                            exact(cur.w[t][2 * p], cur.w[t][2 * p + 1], v);
                        const uintx4 b = {as_u32(v[0] * s2), as_u32(v[1] * s2), as_u32(v[2] * s2), as_u32(v[3] * s2)};
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b),
                                                                        acc[t], 0, 0, 0);
                    }
                }
                cur = nxt;
            }
            // D: lane (n = col, kq), element e: row m = 4 kq + e
#pragma unroll
            for (int t = 0; t < NT; ++t)
                red[wave][t][lane] = acc[t];
            __syncthreads();
            for (int o = tid; o < NT * 256; o += SKINNY_WAVES * 64)
            {
                const int l = o & 63, e = (o >> 6) & 3, t = o >> 8;
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < SKINNY_WAVES; ++w)
                    sum += red[w][t][l][e];
                const int m = 4 * (l >> 4) + e, nn = (block * NT + t) * 16 + (l & 15);
                if (m < M && nn < N)
                    Y[(size_t)m * N + nn] = (half_t)sum;
            }
            __syncthreads(); // the partial tiles are read before the next block's are written
        }
    }

    // Output tiles of 32 WAVES_M WM x 32 WAVES_N WN: WAVES_M x WAVES_N wavefronts of WM x WN MFMA tiles each
    // (v_mfma_f32_32x32x16_f16), K steps of 64 through two LDS buffers, one barrier per step.  A step's operands travel
    // global -> registers -> LDS: the activations as they are (16-byte pieces, a wavefront-wide load takes whole
    // 128-byte lines of 8 rows), the weights dequantised on the way by the thread that fetched them -- the exact
    // integers q - z in fp16 (offset trick) times the scale, one rounding, which is fp16((q - z) * s).  Two sets of
    // staging registers: the loads of step s + 2 are issued ahead of the MFMAs of step s and stored among the MFMAs of
    // step s + 1, so a load has two steps to arrive (with one set a step lasted as long as a load from memory, half a
    // microsecond, whatever M was).  A step runs in quarters (16 values of K): the next quarter's fragments are read
    // from LDS, this quarter's MFMAs issued, and a slice of the next step's pieces unpacked and stored into the other
    // buffer between them.  What a wavefront issues besides MFMAs hardly overlaps its own MFMAs (timing-only builds at
    // 2048 x 8192 x 8192, 8 bits, 256 x 256 tiles on four wavefronts: MFMAs and fragment reads alone 213 us, everything
    // 287, every load served by the same four cache lines 277), so the 256-row tiles run on eight wavefronts, two per
    // SIMD (256 x 256: 563 -> 517 us at 4096 rows; 256 x 128: 171 -> 160 at 1024).  The loads are issued and stored
    // every step, past the end of K at clamped addresses and as zeros: a branch around them would make the compiler wait
    // for every load in flight at the top of the loop.  Tiles are numbered in groups of four tile rows, tile row fastest,
    // and dealt to the eight XCDs in contiguous runs, so that the workgroups in flight together share activations and
    // weights in one L2 (groups of 2, 8 or 16 tile rows measure the same).
    template <int BITS, int WM, int WN, bool TAIL, int WAVES_M, int WAVES_N>
    __global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void wna16_tile_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                             const half_t* __restrict__ S, half_t* __restrict__ Y, int M, int N,
                                                             int K, int tiles_m, int tiles_n, QuantArgs qa)
    {
        constexpr int NW = WAVES_M * WAVES_N, THREADS = 64 * NW; // wavefronts: WAVES_M x WAVES_N
        constexpr int TM = 32 * WAVES_M * WM, TN = 32 * WAVES_N * WN; // rows and columns of the output tile
        constexpr int A_ROWS = THREADS / 8;                   // rows of activations the workgroup fetches per pass
        constexpr int KS = 64;            // values of K per step
        constexpr int PITCH = KS + 8;     // halves per staged row (144 bytes: 16-byte pieces stay aligned)
        constexpr int A_OPERAND = TM * PITCH, W_OPERAND = TN * PITCH; // halves of the staged operands
        constexpr int BUFFER = A_OPERAND + W_OPERAND;
        constexpr int WPP = 128 / BITS;   // weights of a 16-byte piece (inside one group)
        constexpr int PPR = KS / WPP;     // pieces per weight row and step
        constexpr int A_PER = TM / A_ROWS; // pieces of activations per thread and step: piece tid % 8 of rows tid / 8 + 32 i
        constexpr int W_PIECES = TN * PPR;
        // the activations (L2 hits) are fetched one step ahead where a step is long (256-row tiles: a microsecond and
        // more), two steps ahead like the weights otherwise
        constexpr int A_AHEAD = WM >= 4 ? 1 : 2;
        // The barrier of a step stands behind its third quarter where the registers allow it (CARRY: the first fragments
        // of the next step are read during the fourth quarter and carried into the next step; the 256 x 256 tile, whose
        // sums take all 256 accumulation registers, has no room for that and keeps its barrier at the end of the step)
        constexpr bool CARRY = WM * WN < 16 && NW != 8;
        constexpr int SLICES = CARRY ? 3 : 4; // quarters that store pieces of the next step
        constexpr int W_PER = (W_PIECES + THREADS - 1) / THREADS; // pieces of weights per thread and step: piece p % PPR of row p / PPR, p = tid + THREADS j
        extern __shared__ __attribute__((aligned(16))) half_t lds[]; // [buffer][A: TM rows, W: TN rows][PITCH]
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        int tm, tn;
        {
            constexpr int GM = 4;
            const int total = tiles_m * tiles_n, per = total / 8, rem = total % 8;
            const int xcd = (int)blockIdx.x % 8, i = (int)blockIdx.x / 8;
            if (i >= per + (xcd < rem ? 1 : 0))
                return; // (a grid rounded up to whole rounds of the XCDs)
            const int tile = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + i;
            const int per_group = GM * tiles_n;
            const int g = tile / per_group, first_m = g * GM, gm = min(GM, tiles_m - first_m), rr = tile - g * per_group;
            tm = first_m + rr % gm;
            tn = rr / gm;
        }
        const int m0 = tm * TM, n0 = tn * TN;
        const int G = K >> qa.group_shift;
        const size_t row_bytes = (size_t)K * BITS / 8;
        const int steps = (K + KS - 1) / KS;
        const int a_row = tid >> 3, a_k = (tid & 7) * 8;
        // fragments: wavefront (wm, wn) owns rows [32 WM wm, +32 WM) x columns [32 WN wn, +32 WN)
        const int wm = wave / WAVES_N, wn = wave % WAVES_N;
        const int f_row = lane & 31, f_k = (lane >> 5) * 8;

        // what a thread fetches per step, as it arrives: anything computed from it here would be waited for here
        struct Staged
        {
            uintx4 a[A_PER], w[W_PER];
            unsigned short s[W_PER]; // the piece's scale (fp16 bits)
            uint8_t z[W_PER]; // the byte that holds its zero point (widened where it is used: widened here, it would be waited for here)
        };
        // (no zero-point tensor: the byte is fetched all the same, from the scales, and not used -- a branch around the
        // load would make the compiler wait for every load in flight behind it)
        const uint8_t* z_base = qa.zps ? qa.zps : reinterpret_cast<const uint8_t*>(S);
        // piece j of this thread: its weight row (clamped to N - 1), the first of its weights in step `step` (clamped to
        // the last whole piece of the row), its group
        auto w_piece = [&](int step, int j, int& row, int& k, int& n, int& kc, int& g) {
            const int p = min(tid + THREADS * j, W_PIECES - 1);
            row = p / PPR;
            k = step * KS + (p % PPR) * WPP;
            kc = min(k, K - WPP);
            n = min(n0 + row, N - 1);
            g = kc >> qa.group_shift;
        };
        auto fetch_a = [&](int step_raw, Staged& r) {
            const int step = min(step_raw, steps - 1);
#pragma unroll
            for (int i = 0; i < A_PER; ++i)
            {
                const int row = min(m0 + a_row + A_ROWS * i, M - 1), k = min(step * KS + a_k, K - 8);
                r.a[i] = *reinterpret_cast<const uintx4*>(A + (size_t)row * K + k);
            }
        };
        auto fetch_w = [&](int step_raw, Staged& r) {
            const int step = min(step_raw, steps - 1);
#pragma unroll
            for (int j = 0; j < W_PER; ++j)
            {
                int row, k, n, kc, g;
                w_piece(step, j, row, k, n, kc, g);
                r.w[j] = *reinterpret_cast<const uintx4*>(Wq + (size_t)n * row_bytes + (size_t)kc * BITS / 8);
                r.s[j] = reinterpret_cast<const unsigned short*>(S)[(size_t)n * G + g];
                r.z[j] = z_base[(size_t)n * qa.zp_stride + (BITS == 4 ? g >> 1 : g)];
            }
        };
        // piece i of the activations / piece j of the weights of step `step` into its buffer
        auto stage_a = [&](int step, const Staged& r, int i) {
            half_t* a_s = lds + (size_t)(step & 1) * BUFFER;
            // TAIL (K no multiple of 128: a last step of 32, or an odd number of steps, the loop running over an even
            // one): zeros behind the end of K.  (Rows past M repeat row M - 1 and columns past N column N - 1: what they
            // add up is never stored.)
            const bool real = !TAIL || step * KS + a_k < K;
            *reinterpret_cast<uintx4*>(a_s + (a_row + A_ROWS * i) * PITCH + a_k) = real ? r.a[i] : uintx4{0u, 0u, 0u, 0u};
        };
        auto stage_w = [&](int step, const Staged& r, int j) {
            half_t* w_s = lds + (size_t)(step & 1) * BUFFER + A_OPERAND;
            {
                if (W_PIECES % THREADS != 0 && tid + THREADS * j >= W_PIECES)
                    return;
                int row, k, n, kc, g;
                w_piece(step, j, row, k, n, kc, g);
                const int zt = BITS == 4 ? (int)(((uint32_t)r.z[j] >> ((g & 1) * 4)) & 15u) : (int)r.z[j];
                const ExactWeights<BITS> exact(qa.zps ? zt : qa.zp);
                // TAIL: weights of zero behind the end of K
                const uint32_t su = (uint32_t)r.s[j];
                const half2_t s2 = as_half2((!TAIL || k < K) ? __builtin_amdgcn_perm(su, su, 0x05040504u) : 0u);
                const uint32_t ww[4] = {r.w[j].x, r.w[j].y, r.w[j].z, r.w[j].w};
                half_t* dst = w_s + row * PITCH + (k - step * KS);
                if constexpr (BITS == 4)
                {
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                    {
                        half2_t v[4];
                        exact(ww[d], 0u, v); // pairs (0,4) (1,5) (2,6) (3,7) -> order of k
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            v[i] = v[i] * s2;
                        uintx4 o;
                        o.x = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x05040100u);
                        o.y = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x05040100u);
                        o.z = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x07060302u);
                        o.w = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x07060302u);
                        *reinterpret_cast<uintx4*>(dst + 8 * d) = o;
                    }
                }
                else
                {
#pragma unroll
                    for (int d = 0; d < 2; ++d)
                    {
                        half2_t v[4];
                        exact(ww[2 * d], ww[2 * d + 1], v);
                        *reinterpret_cast<uintx4*>(dst + 8 * d) =
                            uintx4{as_u32(v[0] * s2), as_u32(v[1] * s2), as_u32(v[2] * s2), as_u32(v[3] * s2)};
                    }
                }
            }
        };
        // slice q of the pieces of a step (all of them: q < 0): the weights first (ra: the set that holds the step's
        // activations, rw: its weights); a piece of weights counts as three of activations
        constexpr int UNITS = 3 * W_PER + A_PER;
        auto stage = [&](int step, const Staged& ra, const Staged& rw, int q) {
#pragma unroll
            for (int j = 0; j < W_PER; ++j)
                if (q < 0 || 3 * j * SLICES / UNITS == q)
                    stage_w(step, rw, j);
#pragma unroll
            for (int i = 0; i < A_PER; ++i)
                if (q < 0 || (3 * W_PER + i) * SLICES / UNITS == q)
                    stage_a(step, ra, i);
        };
        floatx16 acc[WM][WN];
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0.f;
        // step s: the loads of step s + 2 into the set step s was stored from; then in quarters (16 values of K): the
        // next quarter's fragments, this quarter's MFMAs and, between them, a slice of the next step's pieces on their way
        // into the other buffer (last read before the previous barrier).  With the barrier behind the third quarter
        // every wavefront holds its last fragments of this step and has stored its pieces of the next by then, so the
        // fourth quarter's MFMAs run while the next step's first fragments are read -- nothing waits for LDS behind
        // the barrier.
        half8_t fa_carried[2][WM], fw_carried[2][WN];
        auto read_frags = [&](int s, int kk, half8_t (&fa)[2][WM], half8_t (&fw)[2][WN]) {
            const half_t* a_s = lds + (size_t)(s & 1) * BUFFER;
            const half_t* w_s = a_s + A_OPERAND;
#pragma unroll
            for (int i = 0; i < WM; ++i)
                fa[kk & 1][i] = *reinterpret_cast<const half8_t*>(a_s + ((wm * WM + i) * 32 + f_row) * PITCH + kk * 16 + f_k);
#pragma unroll
            for (int j = 0; j < WN; ++j)
                fw[kk & 1][j] = *reinterpret_cast<const half8_t*>(w_s + ((wn * WN + j) * 32 + f_row) * PITCH + kk * 16 + f_k);
        };
        auto step = [&](int s, Staged& refill, const Staged& ready) {
            if constexpr (A_AHEAD == 1)
                fetch_a(s + 1, refill);
            else
                fetch_a(s + 2, refill);
            fetch_w(s + 2, refill);
            // (the loads stay here, ahead of the MFMAs: among the first quarter's MFMAs they gain nothing at 4096 rows
            // and cost 5 % at a hundred)
            __builtin_amdgcn_sched_barrier(0);
            half8_t fa_local[2][WM], fw_local[2][WN];
            half8_t (&fa)[2][WM] = CARRY ? fa_carried : fa_local;
            half8_t (&fw)[2][WN] = CARRY ? fw_carried : fw_local;
            if constexpr (!CARRY)
                read_frags(s, 0, fa, fw);
#pragma unroll
            for (int kk = 0; kk < KS / 16; ++kk)
            {
                if (kk + 1 < KS / 16)
                    read_frags(s, kk + 1, fa, fw);
                else if constexpr (CARRY)
                    read_frags(s + 1, 0, fa, fw);
#pragma unroll
                for (int i = 0; i < WM; ++i)
#pragma unroll
                    for (int j = 0; j < WN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk & 1][i], fw[kk & 1][j], acc[i][j], 0, 0, 0);
                if (kk < SLICES)
                    stage(s + 1, A_AHEAD == 1 ? refill : ready, ready, kk);
                __builtin_amdgcn_sched_barrier(0);
                if (kk == SLICES - 1)
                    __syncthreads();
            }
        };
        Staged r0, r1;
        fetch_a(0, r0);
        fetch_w(0, r0);
        if constexpr (A_AHEAD == 2)
            fetch_a(1, r1);
        fetch_w(1, r1);
        stage(0, r0, r0, -1);
        __syncthreads();
        if constexpr (CARRY)
            read_frags(0, 0, fa_carried, fw_carried);
        // (no branch around a step or its stores: with an odd number of steps the last one runs past the end of K,
        // where TAIL stores zeros; a step peeled off behind the loop instead had the compiler move all 256 sums of the
        // largest tile through memory)
        for (int s = 0; s < steps; s += 2)
        {
            step(s, r0, r1);
            step(s + 1, r1, r0);
        }
        // D[m][n]: lane l holds column l % 32; element e is row 8 (e / 4) + 4 (l / 32) + e % 4
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
            {
                const int n = n0 + (wn * WN + j) * 32 + (lane & 31);
#pragma unroll
                for (int e = 0; e < 16; ++e)
                {
                    const int m = m0 + (wm * WM + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < M && n < N)
                        Y[(size_t)m * N + n] = (half_t)acc[i][j][e];
                }
            }
    }

    namespace
    {
        template <int BITS, int WM, int WN, bool TAIL, int WAVES_M = 2, int WAVES_N = 2>
        hipError_t launch_wna16_tile_k(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                     const QuantArgs& qa)
        {
            constexpr int NW = WAVES_M * WAVES_N;
            constexpr int TM = 32 * WAVES_M * WM, TN = 32 * WAVES_N * WN;
            constexpr int LDS = 2 * (TM + TN) * (64 + 8) * (int)sizeof(half_t);
            const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
            if ((long long)tiles_m * tiles_n > 0x7fffff00ll)
                return hipErrorInvalidValue;
            auto kernel = &wna16_tile_kernel<BITS, WM, WN, TAIL, WAVES_M, WAVES_N>;
            if (LDS > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, LDS);
                if (e != hipSuccess)
                    return e;
            }
            const int grid = (tiles_m * tiles_n + 7) / 8 * 8; // whole rounds of the XCDs
            hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * NW), LDS, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, M, N, K, tiles_m, tiles_n, qa);
            return hipGetLastError();
        }
    } // namespace

    namespace
    {
        // (K is a multiple of 32; the kernel walks K in pairs of steps of 64)
        template <int BITS, int WM, int WN, int WAVES_M, int WAVES_N>
        hipError_t launch_wna16_tile(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                     const QuantArgs& qa)
        {
            return K % 128 ? launch_wna16_tile_k<BITS, WM, WN, true, WAVES_M, WAVES_N>(stream, A, Wq, S, Y, M, N, K, qa)
                           : launch_wna16_tile_k<BITS, WM, WN, false, WAVES_M, WAVES_N>(stream, A, Wq, S, Y, M, N, K, qa);
        }
    } // namespace

    bool wna16_supported(int M, int N, int K, int bits, int group)
    {
        return M > 0 && N > 0 && K > 0 && (bits == 4 || bits == 8) && (group == 32 || group == 64 || group == 128) && K % group == 0;
    }

    hipError_t launch_wna16_generic(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                    int bits, int group, int zp, const void* zero_points, int num_cu)
    {
        if (!wna16_supported(M, N, K, bits, group))
            return hipErrorInvalidValue;
        QuantArgs qa;
        qa.zps = (const uint8_t*)zero_points;
        qa.group_shift = group == 32 ? 5 : group == 64 ? 6 : 7;
        qa.zp = zp;
        qa.zp_stride = (K / group * bits + 7) / 8;
        // 4-bit weights, a few rows (up to 32 at K = 2048 / 4096, 16 at 8192): the row-streaming MFMA kernel
        if (bits == 4 && M >= 2 && w4a16_mrows_q_supported(M, N, K, qa.group_shift, zero_points != nullptr, num_cu))
            return launch_w4a16_mrows_q(stream, A, Wq, S, Y, M, N, K, qa.group_shift, zp, zero_points, num_cu);
        // 8-bit weights, 2 .. 16 rows at K = 2048 / 4096 / 8192 (up to 32 at 2048 / 4096): the same kernel on bytes
        if (bits == 8 && M >= 2 && w8a16_mrows_q_supported(M, N, K, qa.group_shift, zero_points != nullptr, num_cu))
            return launch_w8a16_mrows_q(stream, A, Wq, S, Y, M, N, K, qa.group_shift, zp, zero_points, num_cu);
        // ... and two or three blocks of 32 rows (of 16 at K = 8192) one block after the other: re-reading the weights per
        // block is faster than the tile kernel below up to there (N = K = 4096: 14 / 16.5 / 23.3 us at 33 / 64 / 96 rows
        // against 31; N = K = 8192: 38 / 56 us at 32 / 48 rows against 62; level at 128 rows resp. N = 22016, behind
        // beyond)
        if (bits == 8 && M > 16)
        {
            const int block = K == 8192 ? 16 : 32;
            const int blocks = (M + block - 1) / block;
            if (blocks <= (N <= 8192 ? 3 : 2) && w8a16_mrows_q_supported(block, N, K, qa.group_shift, zero_points != nullptr, num_cu))
            {
                for (int m0 = 0; m0 < M; m0 += block)
                {
                    // (a last block of one row runs as two: the row before it is computed twice, to the same value)
                    const int rows = M - m0 < block ? M - m0 : block;
                    const int first = rows == 1 ? m0 - 1 : m0;
                    const hipError_t e = launch_w8a16_mrows_q(stream, (const half_t*)A + (size_t)first * K, Wq, S,
                                                              (half_t*)Y + (size_t)first * N, m0 + rows - first, N, K,
                                                              qa.group_shift, zp, zero_points, num_cu);
                    if (e != hipSuccess)
                        return e;
                }
                return hipSuccess;
            }
        }
        if (M <= 16)
        {
            if (M == 1)
            {
                // rows the row-streaming kernel can walk: that kernel
                if (w4a16_gemv_rows_q_supported(1, N, K, qa.group_shift, zero_points != nullptr, num_cu, bits))
                    return launch_w4a16_gemv_rows_q(stream, A, Wq, S, Y, N, K, qa.group_shift, zp, zero_points, num_cu, bits);
                if (bits == 4)
                    launch_wna16_gemv<4, 4, 1>(stream, A, Wq, S, Y, M, N, K, qa, num_cu);
                else
                    launch_wna16_gemv<8, 4, 1>(stream, A, Wq, S, Y, M, N, K, qa, num_cu);
                return hipGetLastError();
            }
            // blocks of two tiles of 16 rows, at most four workgroups per CU
            const int blocks = (N + 31) / 32, cap = num_cu * 4;
            const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
            if (bits == 4)
                hipLaunchKernelGGL((wna16_skinny_kernel<4, 2>), grid, dim3(SKINNY_WAVES * 64), 0, stream, (const half_t*)A,
                                   (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, M, N, K, qa);
            else
                hipLaunchKernelGGL((wna16_skinny_kernel<8, 2>), grid, dim3(SKINNY_WAVES * 64), 0, stream, (const half_t*)A,
                                   (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, M, N, K, qa);
            return hipGetLastError();
        }
        // 256 x 256 (eight wavefronts, 2 x 4, of 128 x 64), 256 x 128 (eight, 4 x 2, of 64 x 64), 128 x 128 or 64 x 64
        // tiles (four wavefronts): the shape with the lowest estimate, in thousandths of the time of one round of
        // 256 x 256 tiles (one tile per CU).  Measured at K = 8192 and 4096 on 256 CUs: a round of 256 x 128 tiles takes
        // 0.60 of that, 128 x 128 tiles 0.45 while every tile has a CU to itself and 0.73 per round of two tiles per CU,
        // 64 x 64 tiles 0.135 + 0.143 per tile and CU (twelve products between 200 and 4096 rows: the estimate picks
        // the fastest of the four measured shapes in each).
        const auto rounds = [&](int tm, int tn, int per_cu) {
            const long long t = (long long)((M + tm - 1) / tm) * ((N + tn - 1) / tn);
            return (t + (long long)num_cu * per_cu - 1) / ((long long)num_cu * per_cu);
        };
        const long long c256 = 1000 * rounds(256, 256, 1), c256n = 600 * rounds(256, 128, 1);
        const long long c128 = rounds(128, 128, 1) == 1 ? 450 : 730 * rounds(128, 128, 2);
        const long long c64 = 135 + 143 * rounds(64, 64, 1);
        if (c256 <= c256n && c256 <= c128 && c256 <= c64)
            return bits == 4 ? launch_wna16_tile<4, 4, 2, 2, 4>(stream, A, Wq, S, Y, M, N, K, qa)
                             : launch_wna16_tile<8, 4, 2, 2, 4>(stream, A, Wq, S, Y, M, N, K, qa);
        if (c256n <= c128 && c256n <= c64)
            return bits == 4 ? launch_wna16_tile<4, 2, 2, 4, 2>(stream, A, Wq, S, Y, M, N, K, qa)
                             : launch_wna16_tile<8, 2, 2, 4, 2>(stream, A, Wq, S, Y, M, N, K, qa);
        if (c128 <= c64)
            return bits == 4 ? launch_wna16_tile<4, 2, 2, 2, 2>(stream, A, Wq, S, Y, M, N, K, qa)
                             : launch_wna16_tile<8, 2, 2, 2, 2>(stream, A, Wq, S, Y, M, N, K, qa);
        return bits == 4 ? launch_wna16_tile<4, 1, 1, 2, 2>(stream, A, Wq, S, Y, M, N, K, qa)
                         : launch_wna16_tile<8, 1, 1, 2, 2>(stream, A, Wq, S, Y, M, N, K, qa);
    }
} // namespace nnf
