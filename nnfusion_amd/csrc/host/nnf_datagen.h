// Deterministic synthetic tensors for the benchmark configurations.
//
// Counter-based: element i of tensor `stream` under `seed` depends only on (seed, stream, i), so
// the host harness, the tests and the CPU baseline all see identical bytes whatever order or
// thread count fills them, with no dependence on a numpy / torch RNG version.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* fp16 (bit patterns) ~ N(mean, stddev), Box-Muller in double, rounded to nearest even */
void nnf_gen_normal_f16(uint64_t seed, uint64_t stream, double mean, double stddev, uint16_t* out, size_t n);
/* fp16 uniform in [lo, hi) */
void nnf_gen_uniform_f16(uint64_t seed, uint64_t stream, double lo, double hi, uint16_t* out, size_t n);
/* fp32 uniform in [lo, hi) */
void nnf_gen_uniform_f32(uint64_t seed, uint64_t stream, double lo, double hi, float* out, size_t n);
/* unsigned 4-bit values uniform in 0..15, packed two per byte (low nibble = even index); n_values even */
void nnf_gen_uniform_u4_packed(uint64_t seed, uint64_t stream, uint8_t* out, size_t n_values);
/* int8 uniform in [lo, hi] inclusive */
void nnf_gen_uniform_i8(uint64_t seed, uint64_t stream, int lo, int hi, int8_t* out, size_t n);
/* IEEE binary16 <-> binary32 conversions (round to nearest even) */
uint16_t nnf_f32_to_f16_bits(float f);
float nnf_f16_bits_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
