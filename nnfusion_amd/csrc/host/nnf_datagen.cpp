#include "nnf_datagen.h"

#include <cmath>
#include <cstring>

namespace
{
    inline uint64_t mix64(uint64_t z)
    {
        z += 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }

    inline uint64_t stream_key(uint64_t seed, uint64_t stream)
    {
        return mix64(mix64(seed) ^ (stream * 0xD1B54A32D192ED03ull));
    }

    inline uint64_t draw(uint64_t key, uint64_t i)
    {
        return mix64(key + i * 0x9E3779B97F4A7C15ull);
    }

    // 53-bit uniform in [0,1)
    inline double u01(uint64_t r)
    {
        return (double)(r >> 11) * (1.0 / 9007199254740992.0);
    }

    uint16_t f2h(float f)
    {
        uint32_t x;
        std::memcpy(&x, &f, 4);
        uint32_t sign = (x >> 16) & 0x8000u;
        uint32_t mag = x & 0x7FFFFFFFu;
        if (mag > 0x7F800000u)
            return (uint16_t)(sign | 0x7E00u);
        if (mag >= 0x477FF000u)
            return (uint16_t)(sign | 0x7C00u);
        if (mag < 0x38800000u)
        {
            // subnormal or zero in fp16: scale so that the integer part is the fp16 mantissa
            float a;
            std::memcpy(&a, &mag, 4);
            float scaled = a * 16777216.0f; // * 2^24, exact
            float r = std::nearbyint(scaled); // default rounding mode: nearest even
            return (uint16_t)(sign | (uint32_t)r);
        }
        uint32_t rounded = mag + 0xFFFu + ((mag >> 13) & 1u);
        return (uint16_t)(sign | ((rounded - 0x38000000u) >> 13));
    }

    float h2f(uint16_t h)
    {
        uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
        uint32_t em = h & 0x7FFFu;
        float out;
        if (em >= 0x7C00u)
        {
            uint32_t bits = sign | 0x7F800000u | ((em & 0x3FFu) << 13);
            std::memcpy(&out, &bits, 4);
        }
        else if (em < 0x0400u)
        {
            out = (float)em * (1.0f / 16777216.0f);
            if (sign)
                out = -out;
        }
        else
        {
            uint32_t bits = sign | ((em << 13) + 0x38000000u);
            std::memcpy(&out, &bits, 4);
        }
        return out;
    }
} // namespace

extern "C" {

uint16_t nnf_f32_to_f16_bits(float f)
{
    return f2h(f);
}

float nnf_f16_bits_to_f32(uint16_t h)
{
    return h2f(h);
}

void nnf_gen_normal_f16(uint64_t seed, uint64_t stream, double mean, double stddev, uint16_t* out, size_t n)
{
    const uint64_t key = stream_key(seed, stream);
    const double two_pi = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
    {
        double u1 = 1.0 - u01(draw(key, 2 * i)); // (0,1]
        double u2 = u01(draw(key, 2 * i + 1));
        double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2);
        out[i] = f2h((float)(mean + stddev * z));
    }
}

void nnf_gen_uniform_f16(uint64_t seed, uint64_t stream, double lo, double hi, uint16_t* out, size_t n)
{
    const uint64_t key = stream_key(seed, stream);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        out[i] = f2h((float)(lo + (hi - lo) * u01(draw(key, i))));
}

void nnf_gen_uniform_f32(uint64_t seed, uint64_t stream, double lo, double hi, float* out, size_t n)
{
    const uint64_t key = stream_key(seed, stream);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        out[i] = (float)(lo + (hi - lo) * u01(draw(key, i)));
}

void nnf_gen_uniform_u4_packed(uint64_t seed, uint64_t stream, uint8_t* out, size_t n_values)
{
    const uint64_t key = stream_key(seed, stream);
    const size_t n_bytes = n_values / 2;
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < n_bytes; ++b)
    {
        uint32_t lo = (uint32_t)(draw(key, 2 * b) >> 60);
        uint32_t hi = (uint32_t)(draw(key, 2 * b + 1) >> 60);
        out[b] = (uint8_t)(lo | (hi << 4));
    }
}

void nnf_gen_uniform_i8(uint64_t seed, uint64_t stream, int lo, int hi, int8_t* out, size_t n)
{
    const uint64_t key = stream_key(seed, stream);
    const uint64_t range = (uint64_t)(hi - lo + 1);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
    {
        uint64_t r = draw(key, i) >> 32;
        out[i] = (int8_t)(lo + (int)((r * range) >> 32));
    }
}

} // extern "C"
