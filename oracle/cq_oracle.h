/*
 * cq_oracle.h — CPU restatement of the reference's quantize/dequantize
 * algorithm (crates/cubek-quant).  TEST INFRASTRUCTURE ONLY: this library is
 * the checker the GPU path is compared against and the timed CPU baseline; the
 * shipped library never links, loads or calls it.
 *
 * All pointers are HOST pointers.  Value tensors are contiguous row-major.
 * `shape` is always the UNPACKED (logical element) shape.
 */
#ifndef CQ_ORACLE_H
#define CQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#include "../include/cubek_quant.h" /* enums and cq_scheme only */

#ifdef __cplusplus
extern "C" {
#endif

/* float formats (bit-level, round-to-nearest-even) */
float cqo_bf16_to_f32(uint16_t h);
uint16_t cqo_f32_to_bf16(float f);
float cqo_f16_to_f32(uint16_t h);
uint16_t cqo_f32_to_f16(float f);

/* scheme */
uint32_t cqo_value_size_bits(uint8_t value);
uint32_t cqo_num_quants(const cq_scheme* scheme);
int cqo_value_range(uint8_t value, float* lo, float* hi);

/* layout (src/layout/scales.rs) */
uint64_t cqo_scale_index(const cq_scheme* scheme, uint32_t rank, const uint64_t* shape,
                         const uint64_t* scale_strides, uint64_t elem);
int cqo_is_block_start(const cq_scheme* scheme, uint32_t rank, const uint64_t* shape,
                       uint64_t elem);

/* bit packing of one word (src/quantize.rs:61-81, src/dequantize.rs:86-118) */
uint32_t cqo_pack_word(const int32_t* codes, uint32_t bits);
void cqo_unpack_word(uint32_t word, uint32_t bits, int32_t* codes);

/* packed-u32 path; words [word_begin, word_end) only (whole tensor: 0, N/nq) */
int cqo_quantize_packed(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                        const void* scale, const uint64_t* scale_strides, void* out_scale,
                        const uint64_t* out_scale_strides, uint32_t* output,
                        const cq_scheme* scheme, uint64_t word_begin, uint64_t word_end);
int cqo_dequantize_packed(const uint32_t* values, uint32_t rank, const uint64_t* shape,
                          const void* params, const uint64_t* scale_strides, void* output,
                          int dtype, const cq_scheme* scheme, uint64_t word_begin,
                          uint64_t word_end);

/* native store path (src/quantize.rs:100-126, src/dequantize.rs:150-167);
 * elements [elem_begin, elem_end), both even for E2M1 */
int cqo_quantize_native(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                        const void* scale, const uint64_t* scale_strides, void* out_scale,
                        const uint64_t* out_scale_strides, uint8_t* output,
                        const cq_scheme* scheme, uint64_t elem_begin, uint64_t elem_end);
int cqo_dequantize_native(const uint8_t* values, uint32_t rank, const uint64_t* shape,
                          const void* params, const uint64_t* scale_strides, void* output,
                          int dtype, const cq_scheme* scheme, uint64_t elem_begin,
                          uint64_t elem_end);

/* fp8 / fp4 element formats used by the native store */
uint8_t cqo_f32_to_e4m3(float f);
float cqo_e4m3_to_f32(uint8_t b);
uint8_t cqo_f32_to_e5m2(float f);
float cqo_e5m2_to_f32(uint8_t b);
uint8_t cqo_f32_to_e2m1(float f);
float cqo_e2m1_to_f32(uint8_t nibble);

/* scale = 2*max|x| / (q_max - q_min) in f32, rounded to `dtype`
 * (tests/suite/symmetric.rs:35-38,156-179); scales are contiguous, typed `dtype` */
int cqo_compute_scales(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                       void* scales, const cq_scheme* scheme);

/* abs-max along one axis, any strides (crates/cubek-reduce/src/instructions/maxabs.rs) */
int cqo_reduce_max_abs(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                       const uint64_t* in_strides, uint32_t axis, void* output,
                       const uint64_t* out_strides);

/* strided quantized tensor -> contiguous, packed along the last dimension
 * (cubecl-std into_contiguous_packed as called at crates/cubek-matmul/src/base.rs:505-529) */
int cqo_into_contiguous_packed(const void* input, uint32_t elem_bytes, uint32_t packing, uint32_t rank,
                               const uint64_t* shape, const uint64_t* in_strides, uint32_t packed_dim,
                               void* output);

/* threaded drivers used for the CPU baseline timing (split the word range) */
int cqo_quantize_packed_mt(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                           const void* scale, const uint64_t* scale_strides, void* out_scale,
                           const uint64_t* out_scale_strides, uint32_t* output,
                           const cq_scheme* scheme, uint64_t word_begin, uint64_t word_end,
                           int threads);
int cqo_dequantize_packed_mt(const uint32_t* values, uint32_t rank, const uint64_t* shape,
                             const void* params, const uint64_t* scale_strides, void* output,
                             int dtype, const cq_scheme* scheme, uint64_t word_begin,
                             uint64_t word_end, int threads);

#ifdef __cplusplus
}
#endif
#endif
