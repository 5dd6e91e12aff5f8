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
//   * wna16_tile_kernel / wna16_tile128_kernel (M > 16): 64 x 64 or, once they fill the chip, 128 x 128 output tiles on
//     v_mfma_f32_32x32x16_f16, K steps of 32 through LDS, the next step's operands fetched into registers while this
//     step's MFMAs run.
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

        // eight consecutive weights of a row starting at k (a multiple of 8), as integers
        template <int BITS>
        __device__ __forceinline__ void load_q8(const uint8_t* __restrict__ row, int k, int (&q)[8])
        {
            if constexpr (BITS == 4)
            {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(row + (k >> 1)); // nibble i = k + i
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    q[i] = (int)((w >> (4 * i)) & 0xFu);
            }
            else
            {
                const uintx2 w = *reinterpret_cast<const uintx2*>(row + k);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    q[i] = (int)((w.x >> (8 * i)) & 0xFFu);
                    q[4 + i] = (int)((w.y >> (8 * i)) & 0xFFu);
                }
            }
        }

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

    // one workgroup of four wavefronts per 64 x 64 output tile (blockIdx.x: column tile, blockIdx.y: row tile)
    template <int BITS>
    __global__ __launch_bounds__(256) void wna16_tile_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                             const half_t* __restrict__ S, half_t* __restrict__ Y, int M, int N,
                                                             int K, QuantArgs qa)
    {
        constexpr int PITCH = 40; // halves per staged row: 32 of K + 8 of padding (80 bytes: 16-byte pieces stay aligned)
        __shared__ __attribute__((aligned(16))) half_t a_s[64 * PITCH];
        __shared__ __attribute__((aligned(16))) half_t w_s[64 * PITCH];
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int m0 = (int)blockIdx.y * 64, n0 = (int)blockIdx.x * 64;
        const int G = K >> qa.group_shift;
        const size_t row_bytes = (size_t)K * BITS / 8;
        // staging: thread t moves eight elements of K (piece t % 4) of row t / 4 of either operand
        const int s_row = tid >> 2, s_k = (tid & 3) * 8;
        const bool a_ok = m0 + s_row < M, w_ok = n0 + s_row < N;
        const half_t* a_src = A + (size_t)min(m0 + s_row, M - 1) * K + s_k;
        const uint8_t* w_row = Wq + (size_t)min(n0 + s_row, N - 1) * row_bytes;
        const int w_n = min(n0 + s_row, N - 1);
        // fragments: wavefront (wm, wn) owns rows [32 wm, +32) x columns [32 wn, +32); lane l holds eight elements of K
        // (block l / 32 of the 16) of row / column l % 32
        const int wm = wave >> 1, wn = wave & 1;
        const int f_row = lane & 31, f_k = (lane >> 5) * 8;

        uintx4 a_next = {0u, 0u, 0u, 0u};
        int q_next[8];
        float s_next = 0.f;
        int z_next = 0;
        auto fetch = [&](int k0) {
            if (a_ok)
                a_next = *reinterpret_cast<const uintx4*>(a_src + k0);
            load_q8<BITS>(w_row, k0 + s_k, q_next);
            const int g = (k0 + s_k) >> qa.group_shift;
            z_next = zero_point_of<BITS>(qa, w_n, g);
            s_next = (float)S[(size_t)w_n * G + g];
        };
        auto stage = [&]() {
            *reinterpret_cast<uintx4*>(a_s + s_row * PITCH + s_k) = a_next; // rows past M stay zero
            half8_t w;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w[i] = w_ok ? (half_t)((float)(q_next[i] - z_next) * s_next) : (half_t)0.f;
            *reinterpret_cast<half8_t*>(w_s + s_row * PITCH + s_k) = w;
        };
        floatx16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = 0.f;
        fetch(0);
        for (int k0 = 0; k0 < K; k0 += 32)
        {
            stage();
            __syncthreads();
            if (k0 + 32 < K)
                fetch(k0 + 32);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
            {
                const half8_t fa = *reinterpret_cast<const half8_t*>(a_s + (wm * 32 + f_row) * PITCH + kk * 16 + f_k);
                const half8_t fw = *reinterpret_cast<const half8_t*>(w_s + (wn * 32 + f_row) * PITCH + kk * 16 + f_k);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fw, acc, 0, 0, 0);
            }
            __syncthreads();
        }
        // D[m][n]: lane l holds column l % 32; element i is row 8 (i / 4) + 4 (l / 32) + i % 4
        const int n = n0 + wn * 32 + (lane & 31);
#pragma unroll
        for (int i = 0; i < 16; ++i)
        {
            const int m = m0 + wm * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
            if (m < M && n < N)
                Y[(size_t)m * N + n] = (half_t)acc[i];
        }
    }

    // 128 x 128 output tiles for products large enough to fill the chip with them: four wavefronts of 64 x 64 (2 x 2 MFMA
    // tiles each), K steps of 32 through two LDS buffers (the next step's operands are fetched into registers ahead of
    // this step's MFMAs and stored behind them: one barrier per step).  A thread stages 16 activations of two rows and
    // dequantises 16 weights of one row per step: the exact integers q - z in fp16 (offset trick) times the scale, one
    // rounding, which is fp16((q - z) * s).  Tiles are numbered in groups of four tile rows, tile row fastest, so that
    // the workgroups in flight together share activations and weights in the caches.
    template <int BITS>
    __global__ __launch_bounds__(256) void wna16_tile128_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S, half_t* __restrict__ Y, int M, int N,
                                                                int K, int tiles_m, int tiles_n, QuantArgs qa)
    {
        constexpr int PITCH = 40;              // halves per staged row: 32 of K + 8 of padding
        constexpr int OPERAND = 128 * PITCH;   // halves of one staged operand
        __shared__ __attribute__((aligned(16))) half_t lds[2][2][OPERAND]; // [buffer][A, W]
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        int tm, tn;
        {
            // workgroups go to the eight XCDs in turn: XCD x takes a contiguous run of tile numbers, so that what its
            // workgroups in flight share stays in its own L2
            constexpr int GM = 4;
            const int total = tiles_m * tiles_n, per = total / 8, rem = total % 8;
            const int xcd = (int)blockIdx.x % 8, i = (int)blockIdx.x / 8;
            const int tile = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + i;
            const int per_group = GM * tiles_n;
            const int g = tile / per_group, first_m = g * GM, gm = min(GM, tiles_m - first_m), rr = tile - g * per_group;
            tm = first_m + rr % gm;
            tn = rr / gm;
        }
        const int m0 = tm * 128, n0 = tn * 128;
        const int G = K >> qa.group_shift;
        const size_t row_bytes = (size_t)K * BITS / 8;
        // staging: activations: piece tid % 4 (8 halves) of rows tid / 4 and 64 + tid / 4; weights: half tid % 2 (16 of the
        // step's 32) of row tid / 2
        const int a_row = tid >> 2, a_k = (tid & 3) * 8;
        const bool a_ok0 = m0 + a_row < M, a_ok1 = m0 + 64 + a_row < M;
        const half_t* a_src0 = A + (size_t)min(m0 + a_row, M - 1) * K + a_k;
        const half_t* a_src1 = A + (size_t)min(m0 + 64 + a_row, M - 1) * K + a_k;
        const int w_row = tid >> 1, w_k = (tid & 1) * 16;
        const int w_n = min(n0 + w_row, N - 1);
        const bool w_ok = n0 + w_row < N;
        const uint8_t* w_src = Wq + (size_t)w_n * row_bytes;
        // fragments: wavefront (wm, wn) owns rows [64 wm, +64) x columns [64 wn, +64)
        const int wm = wave >> 1, wn = wave & 1;
        const int f_row = lane & 31, f_k = (lane >> 5) * 8;

        uintx4 a_next0 = {0u, 0u, 0u, 0u}, a_next1 = {0u, 0u, 0u, 0u}, w_next = {0u, 0u, 0u, 0u};
        float s_next = 0.f;
        int z_next = 0;
        auto fetch = [&](int k0) {
            if (a_ok0)
                a_next0 = *reinterpret_cast<const uintx4*>(a_src0 + k0);
            if (a_ok1)
                a_next1 = *reinterpret_cast<const uintx4*>(a_src1 + k0);
            const int k = k0 + w_k;
            if constexpr (BITS == 4)
            {
                const uintx2 w = *reinterpret_cast<const uintx2*>(w_src + (k >> 1));
                w_next.x = w.x, w_next.y = w.y;
            }
            else
                w_next = *reinterpret_cast<const uintx4*>(w_src + k);
            const int g = k >> qa.group_shift;
            z_next = zero_point_of<BITS>(qa, w_n, g);
            s_next = w_ok ? (float)S[(size_t)w_n * G + g] : 0.f; // (columns past N: weights of zero)
        };
        auto stage = [&](int buf) {
            *reinterpret_cast<uintx4*>(&lds[buf][0][a_row * PITCH + a_k]) = a_next0; // rows past M stay zero
            *reinterpret_cast<uintx4*>(&lds[buf][0][(64 + a_row) * PITCH + a_k]) = a_next1;
            const ExactWeights<BITS> exact(z_next);
            const half_t sh = (half_t)s_next;
            const half2_t s2 = half2_t{sh, sh};
            uintx4 lo, hi; // the 16 weights in order of k, as fp16
            if constexpr (BITS == 4)
            {
                half2_t v[4];
                exact(w_next.x, 0u, v); // pairs (0,4) (1,5) (2,6) (3,7) -> order of k
                for (int i = 0; i < 4; ++i)
                    v[i] = v[i] * s2;
                lo.x = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x05040100u);
                lo.y = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x05040100u);
                lo.z = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x07060302u);
                lo.w = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x07060302u);
                exact(w_next.y, 0u, v);
                for (int i = 0; i < 4; ++i)
                    v[i] = v[i] * s2;
                hi.x = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x05040100u);
                hi.y = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x05040100u);
                hi.z = __builtin_amdgcn_perm(as_u32(v[1]), as_u32(v[0]), 0x07060302u);
                hi.w = __builtin_amdgcn_perm(as_u32(v[3]), as_u32(v[2]), 0x07060302u);
            }
            else
            {
                half2_t v[4];
                exact(w_next.x, w_next.y, v);
                lo = uintx4{as_u32(v[0] * s2), as_u32(v[1] * s2), as_u32(v[2] * s2), as_u32(v[3] * s2)};
                exact(w_next.z, w_next.w, v);
                hi = uintx4{as_u32(v[0] * s2), as_u32(v[1] * s2), as_u32(v[2] * s2), as_u32(v[3] * s2)};
            }
            *reinterpret_cast<uintx4*>(&lds[buf][1][w_row * PITCH + w_k]) = lo;
            *reinterpret_cast<uintx4*>(&lds[buf][1][w_row * PITCH + w_k + 8]) = hi;
        };
        floatx16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0.f;
        fetch(0);
        stage(0);
        __syncthreads();
        int buf = 0;
        for (int k0 = 0; k0 < K; k0 += 32)
        {
            const bool more = k0 + 32 < K;
            if (more)
                fetch(k0 + 32);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
            {
                half8_t fa[2], fw[2];
#pragma unroll
                for (int i = 0; i < 2; ++i)
                {
                    fa[i] = *reinterpret_cast<const half8_t*>(&lds[buf][0][(wm * 64 + i * 32 + f_row) * PITCH + kk * 16 + f_k]);
                    fw[i] = *reinterpret_cast<const half8_t*>(&lds[buf][1][(wn * 64 + i * 32 + f_row) * PITCH + kk * 16 + f_k]);
                }
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fw[j], acc[i][j], 0, 0, 0);
            }
            if (more)
                stage(buf ^ 1); // last read a step ago, before the barrier at its end
            __syncthreads();
            buf ^= 1;
        }
        // D[m][n]: lane l holds column l % 32; element e is row 8 (e / 4) + 4 (l / 32) + e % 4
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
            {
                const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
                for (int e = 0; e < 16; ++e)
                {
                    const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < M && n < N)
                        Y[(size_t)m * N + n] = (half_t)acc[i][j][e];
                }
            }
    }

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
        // ... and up to six blocks of 32 rows (of 16 at K = 8192) one block after the other: the plain tile kernels below
        // spend half a microsecond per 32 values of K whatever M is (N = K = 4096: 68 - 71 us from 33 to 256 rows; a block
        // of 32 rows takes 9.6 us here), so re-reading the weights per block is the faster way up to there
        if (bits == 8 && M > 16)
        {
            const int block = K == 8192 ? 16 : 32;
            const int blocks = (M + block - 1) / block;
            if (blocks <= 6 && w8a16_mrows_q_supported(block, N, K, qa.group_shift, zero_points != nullptr, num_cu))
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
        const int tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
        if ((long long)tiles_m * tiles_n >= num_cu)
        {
            const dim3 grid128((unsigned)(tiles_m * tiles_n));
            if (bits == 4)
                hipLaunchKernelGGL(wna16_tile128_kernel<4>, grid128, dim3(256), 0, stream, (const half_t*)A, (const uint8_t*)Wq,
                                   (const half_t*)S, (half_t*)Y, M, N, K, tiles_m, tiles_n, qa);
            else
                hipLaunchKernelGGL(wna16_tile128_kernel<8>, grid128, dim3(256), 0, stream, (const half_t*)A, (const uint8_t*)Wq,
                                   (const half_t*)S, (half_t*)Y, M, N, K, tiles_m, tiles_n, qa);
            return hipGetLastError();
        }
        const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
        if (grid.y > 65535u)
            return hipErrorInvalidValue;
        if (bits == 4)
            hipLaunchKernelGGL(wna16_tile_kernel<4>, grid, dim3(256), 0, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, M, N, K, qa);
        else
            hipLaunchKernelGGL(wna16_tile_kernel<8>, grid, dim3(256), 0, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, M, N, K, qa);
        return hipGetLastError();
    }
} // namespace nnf
