// cubek_quant_device.hpp — device-side building blocks for kernels that consume
// quantized tensors directly (fuse-on-read), header only, HIP / gfx950.
//
// They are the counterparts of the public #[cube] functions of the reference
// crate, which other kernels (its matmul) inline to dequantize while loading:
//   dequantize_symmetric                  crates/cubek-quant/src/dequantize.rs:20-25
//   dequantize_symmetric_packed_value(s), dequantize_symmetric_packed_value_at   src/dequantize.rs:27-79
//   unpack_q                              src/dequantize.rs:81-118
//   the native-store line of dequantize_symmetric_native_kernel                  src/dequantize.rs:150-167
//   ScalesLayout::{to_source_pos, is_block_start}, scales_layout   src/layout/scales.rs:15-247
//   GlobalScaleLayout (scale of a (batch, row, col) coordinate)
//                                         crates/cubek-matmul/src/components/global/memory/layout.rs:371-455
// Like the reference's functions they are generic over the float type kF the arithmetic is
// carried out in and over the storage type FS of the scales (float, _Float16, __bf16).
// Results are bit-identical to cq_dequantize for the same inputs: y = kF(kF(scale) * kF(code)).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cubek_quant {
namespace device {

// Float type the arithmetic is carried out in (the tensor's type in the reference).
enum class Float { F32, F16, BF16 };

// How the native store holds one value (QuantStore::Native; the U32 store always holds
// two's-complement fields, whatever the value type of the reference).  The one exception is this library's
// extension value CQ_VALUE_E2M1_OCP, whose u32 words hold eight e2m1 nibbles, the same bytes as the native
// store's pairs: decode them with Native::E2M1x2 (dequantize_symmetric_native_value), not as fields.
enum class Native { I8, E4M3, E5M2, E2M1x2 };

// ---- scale parameters --------------------------------------------------------------------

// A stored scale widened to f32 (exact for every storage type).
__host__ __device__ inline float widen(float s) { return s; }
__device__ __forceinline__ float widen(_Float16 s) { return static_cast<float>(s); }
__device__ __forceinline__ float widen(__bf16 s) { return static_cast<float>(s); }

// ---- division by launch-invariant divisors -------------------------------------------------

// n / d and n % d for n < 2^31 as one 32 x 32 -> 64 bit multiplication and a shift (the
// reference's FastDivmod, src/layout/scales.rs:112,153).  With s = ceil(log2 d) and
// magic = floor(2^(31+s) / d) + 1 (which fits 32 bits): n / d == (n * magic) >> (31 + s).
struct FastDivmod {
    uint32_t divisor = 1, magic = 0x80000001u, shift = 31;  // default: division by 1
    FastDivmod() = default;
    // d == 0 (a dimension of an empty tensor, which no position ever indexes) keeps the division by 1
    __host__ __device__ explicit FastDivmod(uint32_t d) : divisor(d == 0 ? 1u : d) {
        if (d == 0) return;
        uint32_t s = 0;
        while ((1ull << s) < d) s++;
        magic = static_cast<uint32_t>((1ull << (31 + s)) / d + 1);
        shift = 31 + s;
    }
    __host__ __device__ uint32_t div(uint32_t n) const {
        return static_cast<uint32_t>((static_cast<uint64_t>(n) * magic) >> shift);
    }
    __host__ __device__ void div_mod(uint32_t n, uint32_t* quotient, uint32_t* remainder) const {
        *quotient = div(n);
        *remainder = n - *quotient * divisor;
    }
};

// ---- scale addressing ------------------------------------------------------------------

// Element index -> scale index, per tensor (rank == 0) or N-D block scaled.
// Plain data: build it on the host with scales_layout(), pass it by value to a kernel.
struct ScalesLayout {
    uint32_t rank = 0;        // 0: one scale for the whole tensor
    FastDivmod shape[8];      // unpacked (element) shape
    FastDivmod block[8];      // block extents, left-padded with 1
    uint64_t strides[8] = {}; // strides of the scales tensor, in elements

    // ScalesLayout::to_source_pos.  Positions below 2^31 (the reference's positions are u32) take
    // the multiply-and-shift divisions, larger ones plain 64-bit arithmetic.
    __host__ __device__ uint64_t to_source_pos(uint64_t pos) const {
        uint64_t scale_offs = 0;
        if (pos < (1ull << 31)) {
            uint32_t offs = static_cast<uint32_t>(pos);
            for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
                uint32_t local;
                shape[d].div_mod(offs, &offs, &local);
                scale_offs += static_cast<uint64_t>(block[d].div(local)) * strides[d];
            }
        } else {
            uint64_t offs = pos;
            for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
                const uint32_t local = static_cast<uint32_t>(offs % shape[d].divisor);
                offs /= shape[d].divisor;
                scale_offs += static_cast<uint64_t>(local / block[d].divisor) * strides[d];
            }
        }
        return scale_offs;
    }
    // ScalesLayout::is_block_start
    __host__ __device__ bool is_block_start(uint64_t pos) const {
        if (rank == 0) return pos == 0;
        uint64_t offs = pos;
        bool start = true;
        for (int d = static_cast<int>(rank) - 1; d >= 0; d--) {
            const uint32_t local = static_cast<uint32_t>(offs % shape[d].divisor);
            offs /= shape[d].divisor;
            start = start && (local % block[d].divisor == 0);
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
        l.shape[d] = FastDivmod(static_cast<uint32_t>(d + 1 == rank ? values_shape[d] * num_quants : values_shape[d]));
        l.block[d] = FastDivmod(d + block_rank < rank ? 1u : block[d + block_rank - rank]);
        l.strides[d] = scales_strides[d];
    }
    return l;
}

// The scale of element (batch, row, col) of a quantized matrix operand: GlobalScaleLayout of the
// reference's matmul, whose block size is a compile-time pair as well.  kBlockRows == 0: one scale
// per tensor.  Dividing by the template constants compiles to shifts (powers of two) or a
// multiplication: a kernel that walks rows and columns never divides.
template <uint32_t kBlockRows, uint32_t kBlockCols>
struct GlobalScaleLayout {
    uint32_t stride_batch = 0, stride_row = 0, stride_col = 0;  // strides of the scales tensor, in elements
    __host__ __device__ uint32_t to_source_pos(uint32_t batch, uint32_t row, uint32_t col) const {
        if constexpr (kBlockRows == 0) {
            return 0;
        } else {
            return batch * stride_batch + (row / kBlockRows) * stride_row + (col / kBlockCols) * stride_col;
        }
    }
};

// ---- rounding --------------------------------------------------------------------------

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

// Two values of a 16-bit kF as they sit in memory (the first in the low half).
template <Float kF>
__device__ __forceinline__ uint32_t pack_pair(float a, float b) {
    static_assert(kF != Float::F32, "pairs are for the 16-bit types");
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    if constexpr (kF == Float::BF16) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32
    } else {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));   // v_cvt_pk_f16_f32, keeps -0
    }
}

// ---- packed (U32) store ----------------------------------------------------------------

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
template <Float kF, class FS>
__device__ __forceinline__ float dequantize_symmetric(float value, FS scale) {
    return round_to<kF>(round_to<kF>(widen(scale)) * value);
}

// dequantize_symmetric_packed_value: one stored word -> 32/kBits values of type kF
// (returned widened to f32; they are exactly representable in kF).
template <Float kF, int kBits, class FS>
__device__ __forceinline__ void dequantize_symmetric_packed_value(uint32_t word, FS scale, float* out) {
    float q[32 / kBits];
    unpack_q<kBits>(word, q);
    const float s = round_to<kF>(widen(scale));
#pragma unroll
    for (int i = 0; i < 32 / kBits; i++) out[i] = round_to<kF>(s * q[i]);
}

// The same values, for a 16-bit kF, as 16/kBits packed pairs ready to be stored or fed to a
// dot-product / matrix instruction: out[i] holds values 2i (low half) and 2i+1 (high half).
// Bit-identical to dequantize_symmetric_packed_value, in about half the instructions:
//   - the fields are biased to unsigned digits (one XOR per word) and separated by masks into
//     the four bytes of a register, where v_cvt_f32_ubyteN turns each into a float (4-bit fields:
//     v_cvt_pk_f32_fp8 turns two at a time, reading a digit as a tiny e4m3 number);
//   - one FMA per value removes the bias and applies the scale: digit * s - bias * s is the
//     exact product s * code (at most 11 + 8 significant bits), so the single rounding of
//     pack_pair is the reference's rounding of F(scale) * F(code);
//   - f16 goes through packed f16 arithmetic instead: the digit is planted in the mantissa of
//     1024 + digit, v_pk_add_f16 removes 1024 + bias exactly and v_pk_mul_f16 multiplies and
//     rounds two values at a time.
// The short sequence needs a "tame" scale: positive, finite and in [2^-100, 2^100) after rounding
// to kF.  For other scales (negative, zero, NaN, huge, tiny) bias * s could overflow, and a zero code
// has to come out as s * (+0) with the scale's sign: they take the plain path.
// dequantize_symmetric_packed_value_pairs() decides per call; a kernel that wants straight-line code
// tests pairs_scale_is_tame() once for many words (say, with a wave-wide vote) and calls
// dequantize_symmetric_packed_value_pairs_tame() directly.
template <Float kF, class FS>
__device__ __forceinline__ bool pairs_scale_is_tame(FS scale) {
    const float s = round_to<kF>(widen(scale));
    // sign clear and exponent field in [27, 227)
    return (__builtin_bit_cast(uint32_t, s) - 0x0d800000u) < (0x71800000u - 0x0d800000u);
}

// Precondition: pairs_scale_is_tame<kF>(scale).
template <Float kF, int kBits, class FS>
__device__ __forceinline__ void dequantize_symmetric_packed_value_pairs_tame(uint32_t word, FS scale, uint32_t* out) {
    static_assert(kF != Float::F32, "pairs are for the 16-bit types");
    static_assert(kBits == 2 || kBits == 4 || kBits == 8, "2, 4 or 8 bits per value");
    constexpr int kN = 32 / kBits;
    constexpr uint32_t kBias = 1u << (kBits - 1);
    const float s = round_to<kF>(widen(scale));
    constexpr uint32_t kBiasWord = kBits == 8 ? 0x80808080u : (kBits == 4 ? 0x88888888u : 0xAAAAAAAAu);
    const uint32_t digits = word ^ kBiasWord;  // field + bias, unsigned
    if constexpr (kF == Float::F16) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const _Float16 sh = static_cast<_Float16>(s);
        const f16x2 s2 = {sh, sh};
        const _Float16 off = static_cast<_Float16>(-(1024.0f + static_cast<float>(kBias)));
        const f16x2 off2 = {off, off};
        constexpr uint32_t kDigit = (1u << kBits) - 1u;
#pragma unroll
        for (int i = 0; i < kN / 2; i++) {
            // values 2i and 2i+1: their digits into the low mantissa bits of two halves holding 1024.0
            const uint32_t lo = (digits >> (2 * i * kBits)) & kDigit;
            const uint32_t hi = (digits >> ((2 * i + 1) * kBits)) & kDigit;
            const uint32_t planted = 0x64006400u | lo | (hi << 16);
            const f16x2 code = __builtin_bit_cast(f16x2, planted) + off2;  // exact
            out[i] = __builtin_bit_cast(uint32_t, s2 * code);              // v_pk_mul_f16, one rounding
        }
    } else {
        const float nbs = -static_cast<float>(kBias) * s;  // exact
        if constexpr (kBits == 8) {
            // bytes are digits already
            const float v0 = __builtin_fmaf(static_cast<float>(digits & 0xffu), s, nbs);
            const float v1 = __builtin_fmaf(static_cast<float>((digits >> 8) & 0xffu), s, nbs);
            const float v2 = __builtin_fmaf(static_cast<float>((digits >> 16) & 0xffu), s, nbs);
            const float v3 = __builtin_fmaf(static_cast<float>(digits >> 24), s, nbs);
            out[0] = pack_pair<kF>(v0, v1);
            out[1] = pack_pair<kF>(v2, v3);
        } else if constexpr (kBits == 4) {
            // even and odd fields as the low nibbles of four bytes each.  A byte 0x0d read as an e4m3 number
            // is d * 2^-9 for every d in 0..15 (denormals, then the first binade, in one linear run), so
            // v_cvt_pk_f32_fp8 turns two digits into floats per instruction; s * 512 takes the 2^-9 back
            typedef float f32x2 __attribute__((ext_vector_type(2)));
            // (mask, then bias: each is one three-operand bit operation on gfx950)
            const uint32_t even = (word & 0x0f0f0f0fu) ^ 0x08080808u, odd = ((word >> 4) & 0x0f0f0f0fu) ^ 0x08080808u;
            const f32x2 e01 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(even), false);
            const f32x2 e23 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(even), true);
            const f32x2 o01 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(odd), false);
            const f32x2 o23 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(odd), true);
            const float s512 = s * 512.0f;  // exact: s < 2^100
            out[0] = pack_pair<kF>(__builtin_fmaf(e01[0], s512, nbs), __builtin_fmaf(o01[0], s512, nbs));
            out[1] = pack_pair<kF>(__builtin_fmaf(e01[1], s512, nbs), __builtin_fmaf(o01[1], s512, nbs));
            out[2] = pack_pair<kF>(__builtin_fmaf(e23[0], s512, nbs), __builtin_fmaf(o23[0], s512, nbs));
            out[3] = pack_pair<kF>(__builtin_fmaf(e23[1], s512, nbs), __builtin_fmaf(o23[1], s512, nbs));
        } else {
            // field j of every byte, j = 0..3: byte b of ((word >> 2j) & 0x03030303) ^ 0x02020202 is the digit of
            // value 4b + j, and as an e4m3 number it is digit * 2^-9 like the nibbles above
            typedef float f32x2 __attribute__((ext_vector_type(2)));
            const float s512 = s * 512.0f;  // exact: s < 2^100
            f32x2 lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t plane = ((word >> (2 * j)) & 0x03030303u) ^ 0x02020202u;
                lo[j] = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(plane), false);
                hi[j] = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(plane), true);
            }
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float v0 = __builtin_fmaf(b < 2 ? lo[0][b & 1] : hi[0][b & 1], s512, nbs);
                const float v1 = __builtin_fmaf(b < 2 ? lo[1][b & 1] : hi[1][b & 1], s512, nbs);
                const float v2 = __builtin_fmaf(b < 2 ? lo[2][b & 1] : hi[2][b & 1], s512, nbs);
                const float v3 = __builtin_fmaf(b < 2 ? lo[3][b & 1] : hi[3][b & 1], s512, nbs);
                out[2 * b] = pack_pair<kF>(v0, v1);
                out[2 * b + 1] = pack_pair<kF>(v2, v3);
            }
        }
    }
}

template <Float kF, int kBits, class FS>
__device__ __forceinline__ void dequantize_symmetric_packed_value_pairs(uint32_t word, FS scale, uint32_t* out) {
    constexpr int kN = 32 / kBits;
    if (pairs_scale_is_tame<kF>(scale)) {
        dequantize_symmetric_packed_value_pairs_tame<kF, kBits>(word, scale, out);
    } else {
        float v[kN];
        dequantize_symmetric_packed_value<kF, kBits>(word, scale, v);
#pragma unroll
        for (int i = 0; i < kN / 2; i++) out[i] = pack_pair<kF>(v[2 * i], v[2 * i + 1]);
    }
}

// dequantize_symmetric_packed_value_at: a word the caller already holds (`position` is its
// index in the packed tensor), its scale looked up through the layout: the scale of the word's
// first element, as the reference indexes its scales view.
template <Float kF, int kBits, class FS>
__device__ __forceinline__ void dequantize_symmetric_packed_value_at(uint64_t position, uint32_t word,
                                                                     const FS* scales, const ScalesLayout& layout,
                                                                     float* out) {
    const uint64_t elem = position * (32 / kBits);
    dequantize_symmetric_packed_value<kF, kBits>(word, scales[layout.to_source_pos(elem)], out);
}

// dequantize_symmetric_packed_values: word `position` of a packed tensor.
template <Float kF, int kBits, class FS>
__device__ __forceinline__ void dequantize_symmetric_packed_values(uint64_t position, const uint32_t* values,
                                                                   const FS* scales, const ScalesLayout& layout,
                                                                   float* out) {
    dequantize_symmetric_packed_value_at<kF, kBits>(position, values[position], scales, layout, out);
}

// ---- native store ----------------------------------------------------------------------

// Values per 32 bits of a native tensor.
template <Native kNative>
constexpr int native_values_per_word() {
    return kNative == Native::E2M1x2 ? 8 : 4;
}

// The values held by 32 bits of a native tensor, element 0 in the low bits: four i8 / e4m3 /
// e5m2 bytes, or eight e2m1 nibbles (element 2k in the low nibble of byte k).  The conversions
// are gfx950 instructions; every stored value is exact in f32.
template <Native kNative>
__device__ __forceinline__ void decode_native(uint32_t word, float* out) {
    if constexpr (kNative == Native::I8) {
        unpack_q<8>(word, out);
    } else if constexpr (kNative == Native::E4M3) {
        out[0] = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 0);
        out[1] = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 1);
        out[2] = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 2);
        out[3] = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 3);
    } else if constexpr (kNative == Native::E5M2) {
        out[0] = __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(word), 0);
        out[1] = __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(word), 1);
        out[2] = __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(word), 2);
        out[3] = __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(word), 3);
    } else {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0);
        const f32x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
        const f32x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2);
        const f32x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
        out[0] = p0[0], out[1] = p0[1], out[2] = p1[0], out[3] = p1[1];
        out[4] = p2[0], out[5] = p2[1], out[6] = p3[0], out[7] = p3[1];
    }
}

// One line of the native dequantize kernel (src/dequantize.rs:150-167): the values of 32 bits of
// a native tensor times one scale, F(scale) * F(q).
template <Float kF, Native kNative, class FS>
__device__ __forceinline__ void dequantize_symmetric_native_value(uint32_t word, FS scale, float* out) {
    constexpr int kN = native_values_per_word<kNative>();
    float q[kN];
    decode_native<kNative>(word, q);
    const float s = round_to<kF>(widen(scale));
#pragma unroll
    for (int i = 0; i < kN; i++) out[i] = round_to<kF>(s * q[i]);  // F(q) is exact: every stored value fits kF
}

// dequantize_symmetric_native_value as packed pairs of a 16-bit kF, as they sit in memory: two values out of
// 32 bits per conversion, one multiplication each (exact in f32: at most 8 significant bits times at most 11),
// one rounding per pair.  The same operations as the plain function, so every scale is taken (negative, zero,
// infinite, NaN).  I8 bytes are the 8-bit fields of the U32 store: dequantize_symmetric_packed_value_pairs<kF, 8>.
template <Float kF, Native kNative, class FS>
__device__ __forceinline__ void dequantize_symmetric_native_value_pairs(uint32_t word, FS scale, uint32_t* out) {
    static_assert(kF != Float::F32, "pairs are for the 16-bit types");
    static_assert(kNative != Native::I8, "I8 bytes: dequantize_symmetric_packed_value_pairs<kF, 8>");
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const float s = round_to<kF>(widen(scale));
    constexpr int kPairs = native_values_per_word<kNative>() / 2;
    f32x2 q[kPairs];
    if constexpr (kNative == Native::E4M3) {
        q[0] = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), false);
        q[1] = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), true);
    } else if constexpr (kNative == Native::E5M2) {
        q[0] = __builtin_amdgcn_cvt_pk_f32_bf8(static_cast<int>(word), false);
        q[1] = __builtin_amdgcn_cvt_pk_f32_bf8(static_cast<int>(word), true);
    } else {
        q[0] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0);
        q[1] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
        q[2] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2);
        q[3] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
    }
#pragma unroll
    for (int i = 0; i < kPairs; i++) {
        float a = s * q[i][0], b = s * q[i][1];
        if constexpr (kF == Float::F16) {
            // pinned: fused with the conversion (v_fma_mixlo_f16, +0 addend) a negative zero product would turn +0
            asm("" : "+v"(a));
            asm("" : "+v"(b));
        }
        out[i] = pack_pair<kF>(a, b);
    }
}

// 32 bits of a native tensor at `position` (in units of 32 bits), scaled by the scale of their first
// element, as the reference's kernel scales a line (the last block extent must be a multiple of the
// values per 32 bits).
template <Float kF, Native kNative, class FS>
__device__ __forceinline__ void dequantize_symmetric_native_values(uint64_t position, const uint32_t* values,
                                                                   const FS* scales, const ScalesLayout& layout,
                                                                   float* out) {
    const uint64_t elem = position * native_values_per_word<kNative>();
    dequantize_symmetric_native_value<kF, kNative>(values[position], scales[layout.to_source_pos(elem)], out);
}

}  // namespace device
}  // namespace cubek_quant
