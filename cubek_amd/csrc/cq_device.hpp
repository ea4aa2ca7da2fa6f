// Device-side building blocks shared by the gfx950 quantize/dequantize kernels.
//
// Arithmetic contract (what the reference's kernels compute, restated for one
// wave): every operation on the tensor's float type F is the f32 operation on
// the widened operands followed by ONE round-to-nearest-even to F.
//   quantize  : code = clamp(rint(F(x / d)), lo, hi)      crates/cubek-quant/src/quantize.rs:19-31
//   pack      : field i at bits [i*bits,(i+1)*bits)        src/quantize.rs:61-81
//   dequantize: y = F(F(scale) * F(code))                  src/dequantize.rs:22-25,86-118
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/cubek_quant.h"

namespace cq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(<kCount-1>) — for
// builtins whose selector operands must be constants.
template <int kBegin, int kCount, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
    if constexpr (kCount > 0) {
        f(std::integral_constant<int, kBegin>{});
        static_for<kBegin + 1, kCount - 1>(f);
    }
}

__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// Streaming accesses: every byte is touched once, so loads and stores carry the
// non-temporal hint.  (CQ_PLAIN_STORES / CQ_PLAIN_LOADS exist for experiments.)
template <class T>
__device__ __forceinline__ T stream_load(const T* p) {
#ifdef CQ_PLAIN_LOADS
    return *p;
#else
    return __builtin_nontemporal_load(p);
#endif
}
template <class T>
__device__ __forceinline__ void stream_store(T v, T* p) {
#ifdef CQ_PLAIN_STORES
    *p = v;
#else
    __builtin_nontemporal_store(v, p);
#endif
}

// ---- element types -------------------------------------------------------
// A "chunk" is 16 bytes of a float tensor: the unit one lane loads or stores.

struct F32 {
    static constexpr int kDtype = CQ_F32;
    static constexpr int kBytes = 4;
    static constexpr int kPerChunk = 4;
    __device__ static __forceinline__ float round(float v) { return v; }
    __device__ static __forceinline__ float load(const void* p, uint64_t i) {
        return static_cast<const float*>(p)[i];
    }
    // an element that is read once (see stream_load)
    __device__ static __forceinline__ float load_once(const void* p, uint64_t i) {
        return stream_load(static_cast<const float*>(p) + i);
    }
    __device__ static __forceinline__ void store(void* p, uint64_t i, float v) {
        static_cast<float*>(p)[i] = v;
    }
    __device__ static __forceinline__ void unpack(u32x4 raw, float* v) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = bits_f32(raw[j]);
    }
    // values already rounded to F
    __device__ static __forceinline__ u32x4 pack(const float* v) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; j++) r[j] = f32_bits(v[j]);
        return r;
    }
};

struct BF16 {
    static constexpr int kDtype = CQ_BF16;
    static constexpr int kBytes = 2;
    static constexpr int kPerChunk = 8;
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, RNE
    }
    __device__ static __forceinline__ float round(float v) {
        return bits_f32(pack2(v, 0.0f) << 16);
    }
    __device__ static __forceinline__ float load(const void* p, uint64_t i) {
        return bits_f32(static_cast<uint32_t>(static_cast<const uint16_t*>(p)[i]) << 16);
    }
    __device__ static __forceinline__ float load_once(const void* p, uint64_t i) {
        return bits_f32(static_cast<uint32_t>(stream_load(static_cast<const uint16_t*>(p) + i)) << 16);
    }
    __device__ static __forceinline__ void store(void* p, uint64_t i, float v) {
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(pack2(v, 0.0f) & 0xffffu);
    }
    __device__ static __forceinline__ void unpack(u32x4 raw, float* v) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[2 * j] = bits_f32(raw[j] << 16);
            v[2 * j + 1] = bits_f32(raw[j] & 0xffff0000u);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float* v) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; j++) r[j] = pack2(v[2 * j], v[2 * j + 1]);
        return r;
    }
};

struct F16 {
    static constexpr int kDtype = CQ_F16;
    static constexpr int kBytes = 2;
    static constexpr int kPerChunk = 8;
    // f32 -> f16 (RNE).  `v` is first pinned as an f32 value of its own: when it is a product, the
    // compiler otherwise fuses the multiply and the conversion into v_fma_mixlo_f16 with a +0
    // addend, and (-0) + (+0) = +0 loses the sign of a negative zero.
    __device__ static __forceinline__ _Float16 narrow(float v) {
        asm("" : "+v"(v));
        return static_cast<_Float16>(v);
    }
    // not pinned: no caller rounds a product that can be a negative zero (scales are positive,
    // quotients come out of inline assembly), and the hot dequantize kernels round a scale per chunk
    __device__ static __forceinline__ float round(float v) { return static_cast<float>(static_cast<_Float16>(v)); }
    __device__ static __forceinline__ float load(const void* p, uint64_t i) {
        return static_cast<float>(static_cast<const _Float16*>(p)[i]);
    }
    __device__ static __forceinline__ float load_once(const void* p, uint64_t i) {
        return static_cast<float>(stream_load(static_cast<const _Float16*>(p) + i));
    }
    __device__ static __forceinline__ void store(void* p, uint64_t i, float v) {
        static_cast<_Float16*>(p)[i] = narrow(v);
    }
    __device__ static __forceinline__ void unpack(u32x4 raw, float* v) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t w = raw[j];  // copy first: bit-casting the vector element in place reads lane 0
            f16x2 h = __builtin_bit_cast(f16x2, w);
            v[2 * j] = static_cast<float>(h[0]);
            v[2 * j + 1] = static_cast<float>(h[1]);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float* v) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // plain casts: pairs become v_cvt_pk_f16_f32, which keeps the sign of zero, and pinning the
            // inputs as narrow() does costs the 4-bit dequantize kernels 8 % (the negative-zero test
            // watches this path too)
            f16x2 h = {static_cast<_Float16>(v[2 * j]), static_cast<_Float16>(v[2 * j + 1])};
            r[j] = __builtin_bit_cast(uint32_t, h);
        }
        return r;
    }
};

// Round an f32 value to a runtime-selected dtype (scale parameters), widened back.
__device__ __forceinline__ float round_to_dtype(int dtype, float v) {
    // both roundings and a select: no branch in the middle of a kernel's arithmetic
    const float as_bf16 = BF16::round(v), as_f16 = F16::round(v);
    return dtype == CQ_F32 ? v : (dtype == CQ_BF16 ? as_bf16 : as_f16);
}
__device__ __forceinline__ float load_dtype(int dtype, const void* p, uint64_t i) {
    if (dtype == CQ_F32) return F32::load(p, i);
    if (dtype == CQ_BF16) return BF16::load(p, i);
    return F16::load(p, i);
}
// The same load in two steps, for kernels that issue all their loads before any arithmetic and learn the type
// at run time.  Step one has no branch on the type (a branch around a load makes the compiler wait for the
// load where the paths meet): two 16-bit loads, the halves of an f32 or twice the same 16-bit value, both
// inside the tensor whatever the type.  Step two widens, behind all loads.
struct RawScale {
    uint32_t lo, hi;
};
__device__ __forceinline__ RawScale load_dtype_raw(int dtype, const void* p, uint64_t i) {
    const bool wide = dtype == CQ_F32;
    const uint16_t* lo = reinterpret_cast<const uint16_t*>(static_cast<const char*>(p) + (i << (wide ? 2 : 1)));
    return RawScale{lo[0], lo[wide ? 1 : 0]};
}
__device__ __forceinline__ float widen_dtype_raw(int dtype, RawScale raw) {
    const float from_f32 = bits_f32(raw.lo | (raw.hi << 16));
    const float from_bf16 = bits_f32(raw.lo << 16);
    const float from_f16 = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(raw.lo)));
    return dtype == CQ_F32 ? from_f32 : (dtype == CQ_BF16 ? from_bf16 : from_f16);
}
__device__ __forceinline__ void store_dtype(int dtype, void* p, uint64_t i, float v) {
    if (dtype == CQ_F32)
        F32::store(p, i, v);
    else if (dtype == CQ_BF16)
        BF16::store(p, i, v);
    else
        F16::store(p, i, v);
}

// ---- cross-lane helpers (64-wide wave, DPP where the pattern allows) -----

// Reads the lane selected by the DPP control.  bound_ctrl with a zero `old`
// lets the compiler fold the move into the consuming ALU instruction
// (v_max_u32_dpp, v_or_b32_dpp); every pattern used here maps active lanes
// onto active lanes, so the zero is never observed.
template <int kCtrl>
__device__ __forceinline__ uint32_t dpp(uint32_t v) {
    return static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(v), kCtrl, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside each 8 lanes
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i inside each 16 lanes

// max over aligned groups of kGroup lanes (kGroup a power of two, 1..64); every
// lane of the group receives the result.  Inputs must be non-negative and not
// NaN: their bit patterns then order like unsigned integers, which keeps the
// butterfly free of float canonicalisation.
template <int kGroup>
__device__ __forceinline__ float group_max(float v) {
    uint32_t b = f32_bits(v);
    if constexpr (kGroup >= 2) b = max(b, dpp<kDppXor1>(b));
    if constexpr (kGroup >= 4) b = max(b, dpp<kDppXor2>(b));
    if constexpr (kGroup >= 8) b = max(b, dpp<kDppHalfMirror>(b));
    if constexpr (kGroup >= 16) b = max(b, dpp<kDppMirror>(b));
    if constexpr (kGroup >= 32) b = max(b, static_cast<uint32_t>(__shfl_xor(static_cast<int>(b), 16, kWave)));
    if constexpr (kGroup >= 64) b = max(b, static_cast<uint32_t>(__shfl_xor(static_cast<int>(b), 32, kWave)));
    return bits_f32(b);
}

// The same with the group size (2^log2 lanes, log2 <= 6) known at run time only; `log2` is the same for every lane.
__device__ __forceinline__ float group_max_rt(float v, uint32_t log2) {
    uint32_t b = f32_bits(v);
    if (log2 >= 1) b = max(b, dpp<kDppXor1>(b));
    if (log2 >= 2) b = max(b, dpp<kDppXor2>(b));
    if (log2 >= 3) b = max(b, dpp<kDppHalfMirror>(b));
    if (log2 >= 4) b = max(b, dpp<kDppMirror>(b));
    if (log2 >= 5) b = max(b, static_cast<uint32_t>(__shfl_xor(static_cast<int>(b), 16, kWave)));
    if (log2 >= 6) b = max(b, static_cast<uint32_t>(__shfl_xor(static_cast<int>(b), 32, kWave)));
    return bits_f32(b);
}

// OR over aligned groups of 2 or 4 lanes (bit-field assembly across lanes).
template <int kGroup>
__device__ __forceinline__ uint32_t group_or(uint32_t v) {
    if constexpr (kGroup >= 2) v |= dpp<kDppXor1>(v);
    if constexpr (kGroup >= 4) v |= dpp<kDppXor2>(v);
    return v;
}

// ---- quantize arithmetic -------------------------------------------------

// Per-launch constants of the value type.
struct QuantParams {
    float lo, hi;         // q_min, q_max
    float width, rwidth;  // q_max - q_min and its correctly rounded reciprocal
    uint32_t unrounded = 0;  // Range::unrounded
    uint32_t keep = 0;    // the flat quantize kernels: codes leave through output_store(keep = true): they stay in the
                          // Infinity Cache for the kernel that reads them next
};
// A store that streams past the caches, or one that is written through the L2 at system scope (sc0 sc1): it leaves
// no dirty line behind in the L2, as a plain store would (which costs the launch 4 - 8 %), but unlike the streaming
// store it leaves the data in the memory-side Infinity Cache.  `keep` is the same for the whole launch: a scalar
// branch.  A relaxed atomic store of 4 or 8 bytes is how the compiler is told the scope; nothing here is atomic
// in any other sense.
template <class T>
__device__ __forceinline__ void output_store(bool keep, T v, T* p) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "codes leave as one or two words per lane");
    if (keep) {
        if constexpr (sizeof(T) == 8)
            __scoped_atomic_store_n(reinterpret_cast<uint64_t*>(p), __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                                    __MEMORY_SCOPE_SYSTEM);
        else
            __scoped_atomic_store_n(reinterpret_cast<uint32_t*>(p), __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED,
                                    __MEMORY_SCOPE_SYSTEM);
    } else {
        stream_store(v, p);
    }
}

// Divisors for which x * rcp(d) stays within 2^-21 relative error of x / d:
// positive, finite, normal and far from the ends of the exponent range (false for NaN).
// Negative divisors (only a caller's own scales can be negative) take the IEEE division:
// the residual steps of the f16 path add zeros of opposite sign, which loses the sign of
// the zero quotient (-0) / d for d < 0.
__device__ __forceinline__ bool divisor_is_tame(float d) {
    // sign clear and exponent field in [27, 227): 2^-100 <= d < 2^100
    return (f32_bits(d) - 0x0d800000u) < (0x71800000u - 0x0d800000u);
}
// abs-max values for which the scale 2*amax/width (width <= 2^17) and its
// divisor are tame: 2^-80 <= amax < 2^80.
__device__ __forceinline__ bool absmax_is_tame(float amax) {
    return (f32_bits(amax) - 0x17800000u) < (0x67800000u - 0x17800000u);
}

// Reference clamp: max(lo, min(x, hi)) with minNum/maxNum, so NaN -> hi.
__device__ __forceinline__ float clamp_code(float r, float lo, float hi) {
    return fmaxf(lo, fminf(r, hi));
}
// The same function in one instruction, on NEGATED operands: v_med3_f32 returns
// min3 when an operand is NaN, so med3(-x, -hi, -lo) = -clamp(x) for numbers and
// -hi for NaN.  Inline asm, because the compiler folds the surrounding negations
// through the intrinsic (valid for numbers only), which would turn NaN into lo.
__device__ __forceinline__ float neg_clamp_of_neg(float neg_x, float neg_hi, float neg_lo) {
    float r;
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(neg_x), "v"(neg_hi), "v"(neg_lo));
    return r;
}

// Reference formula, one element, IEEE division.
template <class F>
__device__ __forceinline__ float quantize_exact(float x, float d, float lo, float hi) {
    return clamp_code(__builtin_rintf(F::round(x / d)), lo, hi);
}

// scale = 2*absmax / (q_max - q_min) in f32
// (crates/cubek-quant/tests/suite/symmetric.rs:35-38,176-177), IEEE division.
__device__ __forceinline__ float scale_from_absmax(float amax, float width) {
    return (2.0f * amax) / width;
}
// The same quotient for tame abs-max values without dividing: q = t*(1/w),
// one FMA for the exact residual t - q*w and one to apply it.  For the nine
// widths in use (2, 3, 12, 14, 15, 254, 255, 896, 114688) the result equals the
// IEEE quotient for every f32 significand (checked exhaustively by the tests).
__device__ __forceinline__ float scale_from_absmax_tame(float amax, const QuantParams& p) {
    const float t = amax + amax;
    const float q = t * p.rwidth;
    const float e = __builtin_fmaf(-q, p.width, t);
    return __builtin_fmaf(e, p.rwidth, q);
}

// Quantize kN values of one block (common divisor d).  The result is the
// NEGATED code of each value as an integer-valued float in [-hi, -lo]
// (bit-identical to -quantize_exact); the packing step undoes the sign for free.
//
// bf16: the correctly rounded bf16 quotient of two bf16 numbers is at least
//   2^-17 (relative) away from every bf16 rounding boundary, so rounding
//   x * rcp(d) (error < 2^-21) to bf16 gives the same bits as rounding x / d.
//   Values far outside [lo,hi] or below 1/4 in magnitude land on the same code
//   either way, so overflow/underflow of the product is harmless.  Clamping
//   before the bf16 rounding is legal: rounding is monotone, lo and hi are bf16.
// f32 : rint(x * rcp(d)) can differ from rint(fl(x / d)) only when the product
//   is within 2^-21 relative of a half-integer; such lanes redo the chunk with
//   IEEE division.  Clamping to [lo-1/4, hi+1/4] first removes the ties that
//   clamp anyway and bounds the window by a per-range constant.
// f16 : the f16 boundaries are too close for x * rcp(d) alone (a quotient of two
//   f16 numbers can sit 2^-23 relative from a boundary), so one residual step
//   follows: t = x*r, e = x - t*d (exact in one FMA up to its rounding), q = t + e*r.
//   q is x/d with a relative error near 2^-44 before its final rounding, and a
//   quotient of two 11-bit significands is at least 2^-36 relative away from
//   every f32 rounding boundary, so q is bit for bit the IEEE f32 quotient.
//   t is clamped to [lo-1, hi+1] first: that leaves t alone wherever the code is
//   not decided by the clamp, and turns an infinite t (infinite x) into a finite
//   one so that the residual is +-inf (clamped like the IEEE quotient), not NaN.
// Negation commutes with every step (multiply, RNE rounding, rint).
// kNegated = false gives the codes themselves: the last rounding takes its operand negated (a source
// modifier), which the conversions to fp8 / fp4 cannot do for theirs.
// kRint = false leaves out the integer rounding (the extension value CQ_VALUE_E2M1_OCP, whose one rounding is the cast
// to e2m1 that follows): the results are the clamped quotients in F.  The bf16 and f16 arguments above hold for the
// quotient itself; the f32 shortcut is about rint and is skipped.  Quotients too small for x * rcp(d) to be trusted
// (below the normal range) are far below 1/4, where every value casts to a zero of its sign.
template <class F, int kN, bool kNegated = true, bool kRint = true>
__device__ __forceinline__ void quantize_values_neg(const float* x, float d, bool d_tame, float lo,
                                                    float hi, float* qn) {
    constexpr float kSign = kNegated ? 1.0f : -1.0f;
    if constexpr (F::kDtype == CQ_BF16) {
        if (d_tame) {
            const float nr = -__builtin_amdgcn_rcpf(d);
            const float nhi = -hi, nlo = -lo;
#pragma unroll
            for (int i = 0; i < kN; i += 2) {
                const float a = neg_clamp_of_neg(x[i] * nr, nhi, nlo);
                const float b = neg_clamp_of_neg(x[i + 1] * nr, nhi, nlo);
                const uint32_t p = BF16::pack2(a, b);
                qn[i] = kSign * bits_f32(p << 16);
                qn[i + 1] = kSign * bits_f32(p & 0xffff0000u);
                if constexpr (kRint) {
                    qn[i] = __builtin_rintf(qn[i]);
                    qn[i + 1] = __builtin_rintf(qn[i + 1]);
                }
            }
            return;
        }
    } else if constexpr (F::kDtype == CQ_F16) {
        if (d_tame) {
            const float nr = -__builtin_amdgcn_rcpf(d);
            const float nhi = -hi, nlo = -lo, nhi_t = -(hi + 1.0f), nlo_t = -(lo - 1.0f);
#pragma unroll
            for (int i = 0; i < kN; i++) {
                const float tn = neg_clamp_of_neg(x[i] * nr, nhi_t, nlo_t);  // -t
                const float e = __builtin_fmaf(tn, d, x[i]);                 // x - t*d
                const float qn1 = __builtin_fmaf(e, nr, tn);                 // -(t + e*r)
                qn[i] = kSign * F16::round(neg_clamp_of_neg(qn1, nhi, nlo));
                if constexpr (kRint) qn[i] = __builtin_rintf(qn[i]);
            }
            return;
        }
    } else if constexpr (F::kDtype == CQ_F32 && kRint) {
        if (d_tame) {
            const float nr = -__builtin_amdgcn_rcpf(d);
            const float nhi_q = -(hi + 0.25f), nlo_q = -(lo - 0.25f);
            float worst = 0.0f;
#pragma unroll
            for (int i = 0; i < kN; i += 2) {
                const float t0 = neg_clamp_of_neg(x[i] * nr, nhi_q, nlo_q);
                const float t1 = neg_clamp_of_neg(x[i + 1] * nr, nhi_q, nlo_q);
                qn[i] = __builtin_rintf(kSign * t0);
                qn[i + 1] = __builtin_rintf(kSign * t1);
                worst = fmaxf(worst, fmaxf(fabsf(t0 - kSign * qn[i]), fabsf(t1 - kSign * qn[i + 1])));
            }
            const float window = (fmaxf(fabsf(lo), fabsf(hi)) + 1.0f) * 0x1p-21f;
            if (worst < 0.5f - window) return;
        }
    }
#pragma unroll
    for (int i = 0; i < kN; i++)
        qn[i] = -kSign * (kRint ? quantize_exact<F>(x[i], d, lo, hi) : clamp_code(F::round(x[i] / d), lo, hi));
}

// The codes of kN values for the stored encoding kEnc: negated integer-valued floats for the two's-complement fields,
// the codes themselves for the float encodings; for e2m1 nibbles a launch may ask for the unrounded quotients
// (`unrounded`, the same for the whole launch: a scalar branch).  kEnc is an Encoding, declared below.
template <class F, int kN, int kEnc>
__device__ __forceinline__ void quantize_codes(const float* x, float d, bool d_tame, float lo, float hi,
                                               bool unrounded, float* qn) {
    if constexpr (kEnc == 3) {  // kEncE2M1
        if (unrounded) {
            quantize_values_neg<F, kN, false, false>(x, d, d_tame, lo, hi, qn);
            return;
        }
    }
    quantize_values_neg<F, kN, kEnc == 0>(x, d, d_tame, lo, hi, qn);
}

// ---- bit packing -----------------------------------------------------------

// Two's-complement bit fields by mask and shift: kN NEGATED integer-valued
// floats -> kN*kBits bits, element 0 in the low bits.  Values outside the field range
// wrap, as `i32 & mask` does in the reference (src/quantize.rs:75).
template <int kBits, int kN>
__device__ __forceinline__ uint32_t pack_fields_neg(const float* qn) {
    static_assert(kN * kBits <= 32, "fields must fit one word");
    constexpr uint32_t kMask = (1u << kBits) - 1u;
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < kN; i++) {
        uint32_t f = static_cast<uint32_t>(-static_cast<int32_t>(qn[i])) & kMask;
        w |= f << (i * kBits);
    }
    return w;
}

// bias pattern: the digit 2^(kBits-1) repeated over `bits` bits (0x8888.., 0x8080.., 0xAAAA..)
template <int kBits>
__host__ __device__ constexpr uint32_t field_bias(int bits) {
    uint32_t b = 0;
    for (int i = 0; i < bits; i += kBits) b |= (1u << (kBits - 1)) << i;
    return b;
}

// kCount NEGATED integer-valued floats, each code inside the field range
// [-2^(kBits-1), 2^(kBits-1)-1], -> kCount*kBits (<= 16) bits of BIASED digits
// (code + 2^(kBits-1)), element 0 lowest, in the low bits of the result; the bits
// above are garbage.  Horner in f32 is exact (all partial sums are integers below
// 2^16) and subtracting from 2^23 + bias leaves the integer in the low mantissa
// bits.  XOR with field_bias turns biased digits into two's-complement fields.
template <int kBits, int kCount>
__device__ __forceinline__ uint32_t pack_biased_neg(const float* cn) {
    static_assert(kBits * kCount <= 16, "exactness needs at most 16 bits per float");
    float u = cn[kCount - 1];
#pragma unroll
    for (int i = kCount - 2; i >= 0; i--) u = __builtin_fmaf(u, static_cast<float>(1 << kBits), cn[i]);
    constexpr float kMagic = 8388608.0f + static_cast<float>(field_bias<kBits>(kBits * kCount));
    return f32_bits(kMagic - u);
}

// The codes of one 16-byte chunk (given negated) as two's-complement fields.  kChunkBits = kN*kBits:
//   64 -> w[0], w[1]; 32 -> w[0]; 16 / 8 -> low bits of w[0], upper bits zero.
// kWide: the value range exceeds the field (E4M3/E5M2 in 8-bit fields), fields wrap.
template <int kBits, int kN, bool kWide>
__device__ __forceinline__ void pack_chunk_neg(const float* c, uint32_t* w) {
    constexpr int kChunkBits = kN * kBits;
    if constexpr (kWide) {
        if constexpr (kChunkBits == 64) {
            w[0] = pack_fields_neg<kBits, 4>(c);
            w[1] = pack_fields_neg<kBits, 4>(c + 4);
        } else {
            w[0] = pack_fields_neg<kBits, kN>(c);
        }
    } else if constexpr (kChunkBits >= 32) {
        constexpr int kPerHalf = 16 / kBits;
#pragma unroll
        for (int j = 0; j < kChunkBits / 32; j++) {
            const uint32_t lo16 = pack_biased_neg<kBits, kPerHalf>(c + 2 * j * kPerHalf);
            const uint32_t hi16 = pack_biased_neg<kBits, kPerHalf>(c + (2 * j + 1) * kPerHalf);
            w[j] = __builtin_amdgcn_perm(hi16, lo16, 0x05040100u) ^ field_bias<kBits>(32);
        }
    } else {
        w[0] = (pack_biased_neg<kBits, kN>(c) & ((1u << kChunkBits) - 1u)) ^ field_bias<kBits>(kChunkBits);
    }
}

// f16, two's-complement fields that hold the whole value range, a tame divisor: quotient, rounding, clamp and
// packing of one chunk (eight values) with the tail in packed f16 arithmetic.  The quotient is the one of
// quantize_values_neg (x * rcp(d), one residual step: within 2^-22 of x / d, which rounds to f16 as x / d does);
// then, two values per instruction: rounded to f16 (v_cvt_pk_f16_f32), clamped to [lo, hi] (integers, so clamp and
// rint commute), and added to 1536 + bias, where f16 numbers are one apart: the sum is rint(q) + bias + 1536 with
// the tie going to the even code (1536 and the bias are even), and its low bits are the biased field, since
// 1536 = 0x6600 has none of them set.  The two values of a pair are taken kBits * (pairs per half word) fields
// apart, so that masks and shifts on whole registers put every field in its place.
// Word layout as pack_chunk_neg<kBits, 8, false>.
template <int kBits>
__device__ __forceinline__ void quantize_pack_f16_tame(const float* x, float d, float lo, float hi, uint32_t* w) {
    static_assert(kBits == 2 || kBits == 4 || kBits == 8, "2, 4 or 8 bits per value");
    const float nr = -__builtin_amdgcn_rcpf(d);
    const float nhi_t = -(hi + 1.0f), nlo_t = -(lo - 1.0f);
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float tn = neg_clamp_of_neg(x[i] * nr, nhi_t, nlo_t);  // -t
        const float e = __builtin_fmaf(tn, d, x[i]);                 // x - t*d
        q[i] = -__builtin_fmaf(e, nr, tn);                           // t + e*r (the negation folds into the conversion)
    }
    constexpr float kMagic = 1536.0f + static_cast<float>(1 << (kBits - 1));
    const _Float16 lo_h = static_cast<_Float16>(lo), hi_h = static_cast<_Float16>(hi), magic_h = static_cast<_Float16>(kMagic);
    const f16x2 lo2 = {lo_h, lo_h}, hi2 = {hi_h, hi_h}, magic2 = {magic_h, magic_h};
    // fields of the pair (a, b): biased, in the low bits of the two halves
    const auto fields = [&](int a, int b) {
        f16x2 h = {static_cast<_Float16>(q[a]), static_cast<_Float16>(q[b])};
        h = __builtin_elementwise_max(lo2, __builtin_elementwise_min(h, hi2));  // NaN -> hi, as the other paths
        return __builtin_bit_cast(uint32_t, h + magic2);
    };
    constexpr uint32_t kMask = ((1u << kBits) - 1u) * 0x00010001u;
    if constexpr (kBits == 8) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t a = fields(4 * j, 4 * j + 2) & kMask, b = fields(4 * j + 1, 4 * j + 3) & kMask;
            w[j] = (a | (b << 8)) ^ field_bias<8>(32);
        }
    } else {
        uint32_t v = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) v |= (fields(k, k + 4) & kMask) << (k * kBits);
        if constexpr (kBits == 4)
            w[0] = v ^ field_bias<4>(32);
        else
            w[0] = ((v | (v >> 8)) & 0xffffu) ^ field_bias<2>(16);
    }
}

// Sign-extended field i of a word (v_bfe_i32).
template <int kBits>
__device__ __forceinline__ float unpack_field(uint32_t w, int i) {
    int32_t s = static_cast<int32_t>(w << (32 - kBits - i * kBits)) >> (32 - kBits);
    return static_cast<float>(s);
}

// ---- stored encodings --------------------------------------------------------
// How one quantized value is stored.  kEncInt: two's-complement field (the U32
// store of every value type, and the native i8 store, whose bytes coincide with
// 8-bit fields).  The float encodings are the native store's e4m3 / e5m2 bytes
// and e2m1 nibbles (element 2k in the low nibble), produced by the gfx950
// conversion instructions from the already rounded and clamped integer, as the
// reference's `Q::cast_from(clamp(round(x/scale)))` does (src/quantize.rs:33-43).
enum Encoding : int { kEncInt = 0, kEncE4M3 = 1, kEncE5M2 = 2, kEncE2M1 = 3 };

template <int kEnc>
constexpr int encoding_bits(int int_bits) {
    return kEnc == kEncInt ? int_bits : (kEnc == kEncE2M1 ? 4 : 8);
}

// kN integer-valued floats (the codes themselves, not negated) -> kN stored values, same word layout as
// pack_chunk_neg.
template <int kEnc, int kN>
__device__ __forceinline__ void encode_chunk(const float* q, uint32_t* w) {
    if constexpr (kEnc == kEncE2M1) {
        uint32_t r = 0;
        static_for<0, kN / 2>([&](auto byte) {
            constexpr int b = decltype(byte)::value;
            r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, q[2 * b], q[2 * b + 1], 1.0f, b);
        });
        w[0] = r;
    } else {
#pragma unroll
        for (int j = 0; j < kN / 4; j++) {
            int r = 0;
            if constexpr (kEnc == kEncE4M3) {
                r = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j], q[4 * j + 1], r, false);
                r = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j + 2], q[4 * j + 3], r, true);
            } else {
                r = __builtin_amdgcn_cvt_pk_bf8_f32(q[4 * j], q[4 * j + 1], r, false);
                r = __builtin_amdgcn_cvt_pk_bf8_f32(q[4 * j + 2], q[4 * j + 3], r, true);
            }
            w[j] = static_cast<uint32_t>(r);
        }
    }
}

// Stored values 0..kCount-1 of a word as floats.
template <int kEnc, int kBits, int kCount>
__device__ __forceinline__ void decode_fields(uint32_t w, float* v) {
    static_for<0, kCount>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        if constexpr (kEnc == kEncInt) {
            v[i] = unpack_field<kBits>(w, i);
        } else if constexpr (kEnc == kEncE4M3) {
            v[i] = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(w), i);
        } else if constexpr (kEnc == kEncE5M2) {
            v[i] = __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(w), i);
        } else if constexpr ((i & 1) == 0) {
            f32x2 p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, i / 2);
            v[i] = p[0];
            v[i + 1] = p[1];
        }
    });
}

}  // namespace cq
