// cubek_quant_device.hpp — device-side building blocks for kernels that consume
// quantized tensors directly (fuse-on-read), header only, HIP / gfx950.
//
// They are the counterparts of the public #[cube] functions of the reference
// crate, which other kernels (its matmul) inline to dequantize while loading:
//   dequantize_symmetric                  crates/cubek-quant/src/dequantize.rs:20-25
//   dequantize_symmetric_packed_value(s), dequantize_symmetric_packed_value_at   src/dequantize.rs:27-79
//   unpack_q                              src/dequantize.rs:81-118
//   ScalesLayout::{to_source_pos, is_block_start}, scales_layout   src/layout/scales.rs:15-247
// Results are bit-identical to cq_dequantize for the same inputs.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cubek_quant {
namespace device {

// Float type the arithmetic is carried out in (the tensor's type in the reference).
enum class Float { F32, F16, BF16 };

// Element index -> scale index, per tensor (rank == 0) or N-D block scaled.
// Plain data: fill it on the host, pass it by value to a kernel.
struct ScalesLayout {
    uint32_t rank = 0;        // 0: one scale for the whole tensor
    uint32_t shape[8] = {};   // unpacked (element) shape
    uint32_t block[8] = {};   // block extents, left-padded with 1
    uint64_t strides[8] = {}; // strides of the scales tensor, in elements

    // ScalesLayout::to_source_pos
    __host__ __device__ uint64_t to_source_pos(uint64_t pos) const {
        uint64_t offs = pos, scale_offs = 0;
        for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
            const uint32_t local = static_cast<uint32_t>(offs % shape[d]);
            offs /= shape[d];
            scale_offs += static_cast<uint64_t>(local / block[d]) * strides[d];
        }
        return scale_offs;
    }
    // ScalesLayout::is_block_start
    __host__ __device__ bool is_block_start(uint64_t pos) const {
        if (rank == 0) return pos == 0;
        uint64_t offs = pos;
        bool start = true;
        for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
            const uint32_t local = static_cast<uint32_t>(offs % shape[d]);
            offs /= shape[d];
            start = start && (local % block[d] == 0);
        }
        return start;
    }
};

// scales_layout (src/layout/scales.rs:220-247), host side: the layout of the scales that belong
// to a quantized tensor.
//   values_shape   : shape of the QUANTIZED tensor (its last dimension counts stored elements)
//   num_quants     : values per stored element (the last dimension is multiplied by it)
//   scales_strides : strides of the scales tensor, in elements
//   block          : block size per trailing dimension, block_rank entries (0: one scale per tensor);
//                    left-padded with 1 up to the tensor rank, as BlockSize::to_dim_vec does
inline ScalesLayout scales_layout(const uint64_t* values_shape, uint32_t rank, uint32_t num_quants,
                                  const uint64_t* scales_strides, const uint8_t* block, uint32_t block_rank) {
    ScalesLayout l;
    if (block_rank == 0) return l;  // per tensor
    l.rank = rank;
    for (uint32_t d = 0; d < rank; d++) {
        l.shape[d] = static_cast<uint32_t>(d + 1 == rank ? values_shape[d] * num_quants : values_shape[d]);
        l.block[d] = d + block_rank < rank ? 1u : block[d + block_rank - rank];
        l.strides[d] = scales_strides[d];
    }
    return l;
}

// Round an f32 value to `kF` (round-to-nearest-even), widened back to f32.
template <Float kF>
__device__ __forceinline__ float round_to(float v) {
    if constexpr (kF == Float::F32) {
        return v;
    } else if constexpr (kF == Float::F16) {
        // pin `v` first: fused with a preceding multiply (v_fma_mixlo_f16, +0 addend) the conversion
        // would turn a negative zero product into +0
        asm("" : "+v"(v));
        return static_cast<float>(static_cast<_Float16>(v));
    } else {
        return static_cast<float>(static_cast<__bf16>(v));
    }
}

// unpack_q: the 32/kBits two's-complement fields of a word, element 0 in the low bits.
template <int kBits>
__device__ __forceinline__ void unpack_q(uint32_t word, float* out) {
    static_assert(kBits == 2 || kBits == 4 || kBits == 8, "2, 4 or 8 bits per value");
#pragma unroll
    for (int i = 0; i < 32 / kBits; i++) {
        const int32_t s = static_cast<int32_t>(word << (32 - kBits - i * kBits)) >> (32 - kBits);
        out[i] = static_cast<float>(s);
    }
}

// dequantize_symmetric: x = F(scale) * x_q, computed in kF.
template <Float kF>
__device__ __forceinline__ float dequantize_symmetric(float value, float scale) {
    return round_to<kF>(round_to<kF>(scale) * value);
}

// dequantize_symmetric_packed_value: one stored word -> 32/kBits values of type kF
// (returned widened to f32; they are exactly representable in kF).
template <Float kF, int kBits>
__device__ __forceinline__ void dequantize_symmetric_packed_value(uint32_t word, float scale, float* out) {
    float q[32 / kBits];
    unpack_q<kBits>(word, q);
    const float s = round_to<kF>(scale);
#pragma unroll
    for (int i = 0; i < 32 / kBits; i++) out[i] = round_to<kF>(s * q[i]);
}

// dequantize_symmetric_packed_value_at: a word the caller already holds (`position` is its
// index in the packed tensor), its scale looked up through the layout (`scales` holds f32
// parameters): the scale of the word's first element, as the reference indexes its scales view.
template <Float kF, int kBits>
__device__ __forceinline__ void dequantize_symmetric_packed_value_at(uint64_t position, uint32_t word,
                                                                     const float* scales, const ScalesLayout& layout,
                                                                     float* out) {
    const uint64_t elem = position * (32 / kBits);
    dequantize_symmetric_packed_value<kF, kBits>(word, scales[layout.to_source_pos(elem)], out);
}

// dequantize_symmetric_packed_values: word `position` of a packed tensor.
template <Float kF, int kBits>
__device__ __forceinline__ void dequantize_symmetric_packed_values(uint64_t position, const uint32_t* values,
                                                                   const float* scales, const ScalesLayout& layout,
                                                                   float* out) {
    dequantize_symmetric_packed_value_at<kF, kBits>(position, values[position], scales, layout, out);
}

}  // namespace device
}  // namespace cubek_quant
