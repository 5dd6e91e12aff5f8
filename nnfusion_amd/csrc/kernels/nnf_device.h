// Device-side helpers shared by the gfx950 kernels: vector types, int4 -> fp16 unpacking,
// wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace nnf
{
    typedef _Float16 half_t;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
    typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    typedef float floatx4 __attribute__((ext_vector_type(4)));
    typedef float floatx16 __attribute__((ext_vector_type(16)));
    typedef int intx4 __attribute__((ext_vector_type(4)));
    typedef int intx16 __attribute__((ext_vector_type(16)));
    typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
    typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));

    constexpr int WAVE = 64;

    __device__ __forceinline__ half2_t as_half2(uint32_t u)
    {
        return __builtin_bit_cast(half2_t, u);
    }
    __device__ __forceinline__ uint32_t as_u32(half2_t h)
    {
        return __builtin_bit_cast(uint32_t, h);
    }

    // One 32-bit word holds eight 4-bit weights q0..q7 (q_i at bits 4i..4i+3, i.e. k = i within
    // the word).  fp16 0x6400 is 1024.0 with an ulp of 1, so (nibble | 0x6400) is 1024 + q and a
    // nibble four bits higher gives 1024 + 16 q; both are turned into the exact integer (q - zp)
    // with one packed op.  Output pairs are (q0,q4) (q1,q5) (q2,q6) (q3,q7): the activation
    // operand is stored in the same order (see permute_a8).
    //   c_lo = -(1024 + zp)  (packed),  c_hi = -(64 + zp)  (packed),  sixteenth = 1/16 (packed)
    struct DequantConst
    {
        half2_t c_lo, c_hi, sixteenth;
    };

    __device__ __forceinline__ DequantConst make_dequant_const(int zp)
    {
        DequantConst c;
        half_t lo = (half_t)(-(1024.0f + (float)zp));
        half_t hi = (half_t)(-(64.0f + (float)zp));
        c.c_lo = half2_t{lo, lo};
        c.c_hi = half2_t{hi, hi};
        c.sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
        return c;
    }

    __device__ __forceinline__ void dequant8(uint32_t w, const DequantConst& c, half2_t out[4])
    {
        const uint32_t MAGIC = 0x64006400u;
        uint32_t w8 = w >> 8;
        half2_t lo0 = as_half2((w & 0x000F000Fu) | MAGIC);
        half2_t hi0 = as_half2((w & 0x00F000F0u) | MAGIC);
        half2_t lo1 = as_half2((w8 & 0x000F000Fu) | MAGIC);
        half2_t hi1 = as_half2((w8 & 0x00F000F0u) | MAGIC);
        out[0] = lo0 + c.c_lo;                                        // (q0, q4) - zp
        out[1] = __builtin_elementwise_fma(hi0, c.sixteenth, c.c_hi); // (q1, q5) - zp
        out[2] = lo1 + c.c_lo;                                        // (q2, q6) - zp
        out[3] = __builtin_elementwise_fma(hi1, c.sixteenth, c.c_hi); // (q3, q7) - zp
    }

    // Reorder eight consecutive fp16 activations a0..a7 (as four 32-bit words) into the pair
    // order produced by dequant8: (a0,a4) (a1,a5) (a2,a6) (a3,a7).
    __device__ __forceinline__ uintx4 permute_a8(uintx4 a)
    {
        uintx4 r;
        // v_perm_b32(S0, S1, sel): byte selectors 0-3 pick from S1, 4-7 from S0
        r.x = __builtin_amdgcn_perm(a.z, a.x, 0x05040100u); // lo(a.x)=a0, lo(a.z)=a4
        r.y = __builtin_amdgcn_perm(a.z, a.x, 0x07060302u); // hi(a.x)=a1, hi(a.z)=a5
        r.z = __builtin_amdgcn_perm(a.w, a.y, 0x05040100u); // a2, a6
        r.w = __builtin_amdgcn_perm(a.w, a.y, 0x07060302u); // a3, a7
        return r;
    }

    __device__ __forceinline__ float dot2(half2_t a, half2_t b, float c)
    {
        return __builtin_amdgcn_fdot2(a, b, c, false);
    }

    // Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
    // outstanding global load (vmcnt(0)), which would drain software-pipelined prefetches.
    __device__ __forceinline__ void lds_barrier()
    {
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }

    // f(integral_constant<int, I>) for I = BEGIN .. END-1: for bodies that need I as a compile-time constant
    // (instruction offsets, wait counts)
    template <int BEGIN, int END, class F>
    __device__ __forceinline__ void unroll_for(F&& f)
    {
        if constexpr (BEGIN < END)
        {
            f(std::integral_constant<int, BEGIN>{});
            unroll_for<BEGIN + 1, END>(f);
        }
    }

    // 128-bit LDS read that the compiler's wait-count insertion does not see.  The compiler waits for ALL
    // LDS reads in flight (lgkmcnt(0)) ahead of the first use of any of them once reads issued in different
    // loop iterations are pending; with these, fragments for the next MFMA group stay in flight while the
    // current group is issued.  The value is valid only after lds_wait<N>() on it, N = number of LDS
    // operations issued after the read (LDS operations complete in order).
    template <int OFFSET, class V>
    __device__ __forceinline__ void lds_read_b128_nowait(V& dst, uint32_t lds_addr)
    {
        static_assert(sizeof(V) == 16 && OFFSET >= 0 && OFFSET < 65536, "ds_read_b128 with a 16-bit offset");
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(lds_addr), "n"(OFFSET) : "memory");
    }
    // s_waitcnt lgkmcnt(N); `first` is tied to the wait, `also` (values read before it) to `first`'s
    // position through the order of volatile statements: none of them can be used ahead of the wait.
    template <int N, class V>
    __device__ __forceinline__ void lds_wait(V& first)
    {
        static_assert(N >= 0 && N <= 15, "lgkmcnt is four bits wide");
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(first) : "n"(N) : "memory");
    }
    template <class V>
    __device__ __forceinline__ void lds_wait_also(V& v)
    {
        asm volatile("" : "+v"(v));
    }
    // Activation rows into MFMA operand registers by way of LDS.  A lane of a 16-row MFMA operand wants 16-byte pieces
    // that lie 64 bytes apart in its row, so a load straight into the registers touches two lines of every row for
    // 32 bytes each, four times over; the memory pipeline's time goes by the lines a load touches.  Instead a block of
    // 16 rows x 256 bytes is fetched as whole lines (four wavefront-wide loads of 4 rows x 256 bytes, global -> LDS) and
    // read from LDS in operand order.  Layout of a block: row r at 256 r, its 16 pieces XORed with r (conflict-free
    // 128-bit reads: the 16 lanes of a row quad hit 16 different pieces).
    constexpr int ROW_BLOCK_BYTES = 4096;
    // issue the four loads: row `first_row + r` (clamped to last_row) of a row-major matrix (row_bytes per row), bytes
    // [byte0, byte0 + 256)
    __device__ __forceinline__ void row_block_fetch(const uint8_t* base, size_t row_bytes, int first_row, int last_row, size_t byte0,
                                                    uint8_t* block, int lane)
    {
#pragma unroll
        for (int c = 0; c < 4; ++c)
        {
            const int r = c * 4 + (lane >> 4);
            const int piece = (lane & 15) ^ r;
            const uint8_t* src = base + (size_t)min(first_row + r, last_row) * row_bytes + byte0 + piece * 16;
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                             (void __attribute__((address_space(3)))*)(block + c * 1024), 16, 0, 0);
        }
    }
    // piece p (0 .. 15) of row `row` of a landed block
    __device__ __forceinline__ uintx4 row_block_piece(const uint8_t* block, int row, int p)
    {
        return *reinterpret_cast<const uintx4*>(block + row * 256 + ((p ^ row) << 4));
    }
    // vmcnt-only wait (gfx9 encoding)
    __device__ __forceinline__ constexpr int vmcnt_only(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

    __device__ __forceinline__ uint32_t lds_address(const void* p)
    {
        return (uint32_t)(uintptr_t)(const void __attribute__((address_space(3)))*)p;
    }

    // fp32 value -> fp16, as two roundings (the value is first a rounded fp32).  Without the opaque
    // asm the compiler folds a preceding fp32 multiply into v_fma_mixlo_f16, which rounds the exact
    // product once, straight to fp16, and differs from the two-step result on ties.
    __device__ __forceinline__ half_t f32_to_f16_two_step(float v)
    {
        asm volatile("" : "+v"(v));
        return (half_t)v;
    }

    // sum over the four lanes of a quad (lanes 4i .. 4i+3), in every lane; two DPP moves
    __device__ __forceinline__ float quad_sum(float v)
    {
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false)); // 1,0,3,2
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false)); // 2,3,0,1
        return v;
    }

    // sum over a row of 16 lanes (lanes 16i .. 16i+15), in every lane; four DPP row rotations
    // ---- element-wise tail of a fused product, on fp16 tensors as the unfused graph holds them -------------------
    // the kernels' view of nnf::GemvFusion (nnf_launch.h)
    struct GemvFusionArgs
    {
        const half_t* gamma;
        const float* rstd;
        const half_t* bias;
        const half_t* residual;
        float rms_eps; // gamma without rstd: the kernel computes rsqrt(mean(a^2) + rms_eps) of its activation row itself
    };
    // a * b rounded to fp32, as a value of its own: a conversion to fp16 that follows then rounds a second time wherever it
    // is compiled.  (Left to the compiler, product and conversion may or may not become one mixed-precision instruction
    // that rounds once: two kernels that must agree bit for bit -- the reduction pass and the kernels that add their ranges
    // up themselves -- would differ in the last fp16 bit now and then.)
    __device__ __forceinline__ float f32_product(float a, float b)
    {
        float v = a * b;
        asm volatile("" : "+v"(v));
        return v;
    }
    // y = fp16(sum) (+ bias[n]) (+ residual[at]), each step rounded to fp16
    __device__ __forceinline__ half_t finish_bias_residual(float sum, const half_t* bias, int n, const half_t* residual, size_t at)
    {
        half_t y = (half_t)sum;
        if (bias)
            y = (half_t)((float)y + (float)bias[n]);
        if (residual)
            y = (half_t)((float)y + (float)residual[at]);
        return y;
    }
    // fp16(SiLU(g) * u) of the fp16-rounded gate and up products
    __device__ __forceinline__ half_t finish_silu_gate(float gate_sum, float up_sum)
    {
        const float g = (float)(half_t)gate_sum, u = (float)(half_t)up_sum;
        return (half_t)(g * (1.0f / (1.0f + __expf(-g))) * u);
    }

    __device__ __forceinline__ float row16_sum(float v)
    {
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, false)); // row_ror:8
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, false)); // row_ror:4
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xF, 0xF, false)); // row_ror:2
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xF, 0xF, false)); // row_ror:1
        return v;
    }

    __device__ __forceinline__ float wave_sum(float v)
    {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1)
            v += __shfl_xor(v, off, WAVE);
        return v;
    }
} // namespace nnf
