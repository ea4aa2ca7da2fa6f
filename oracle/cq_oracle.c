/*
 * cq_oracle.c — scalar CPU restatement of the reference's quantize/dequantize
 * algorithm.  TEST INFRASTRUCTURE ONLY (checker + timed CPU baseline); nothing
 * in the shipped library may link, load or call it.
 *
 * Reference files followed (relative to crates/cubek-quant/):
 *   src/quantize.rs, src/dequantize.rs, src/layout/scales.rs, src/lib.rs:20-33,
 *   tests/suite/symmetric.rs:35-38,156-179 (scale rule).
 *
 * Arithmetic model.  The reference computes in the tensor's float type F
 * (f32 | f16 | bf16).  Here every F operation is "the f32 operation on the
 * widened operands, rounded once to F with round-to-nearest-even"; for
 * division and multiplication of 8- or 11-bit significands this equals the
 * correctly rounded F result because f32 carries >= 2p+2 bits.
 *
 * How each function is pinned (tests/test_oracle_*.py; none of the pins retypes the formula):
 *   float conversions          torch / numpy CPU conversions, nearest-value table search
 *   cqo_scale_index, cqo_is_block_start   brute force over small N-D shapes
 *   cqo_pack_word, cqo_unpack_word        exhaustive over fields and positions
 *   cqo_quantize_packed, cqo_dequantize_packed   exact-rational fixtures (tests/golden/),
 *                              hand-derived known answers, torch CPU bf16 arithmetic
 *   cqo_quantize_native, cqo_dequantize_native   exact-rational fixtures of all five native
 *                              value types (minifloats built from their bit fields), hand-written
 *                              byte-level known answers (e2m1 nibbles, every i8 code), identities
 *                              with the packed store, torch CPU float8 conversions
 *   cqo_compute_scales, cqo_reduce_max_abs        numpy, exact rationals, permutation invariance
 *
 * Decisions.  The reference delegates these to its JIT dependency (cubecl, not in the
 * reference tree) and its own tests do not observe them; no check can pin them, so they
 * are fixed here by decision and stated as such wherever results are documented:
 *   - round()   = round-half-to-even (rint);
 *   - clamp()   = max(lo, min(x, hi)) with IEEE minNum/maxNum: NaN -> hi;
 *   - value ranges and num_quants as listed in cqo_value_range/cqo_num_quants;
 *   - float -> e4m3 / e5m2 / e2m1 casts round to nearest, ties to the even code;
 *   - E2M1 native bytes hold element 2k in the low nibble, 2k+1 in the high;
 *   - abs-max ignores NaN elements (Rust f32::max in the reference's test).
 * Given these decisions, every function below is pinned as listed above.
 *
 * Extension.  CQ_VALUE_E2M1_OCP (OCP microscaling FP4 without the reference's integer rounding) has no
 * counterpart in the reference, so there is no parity to speak of; its arm here defines what the kernels must
 * produce, and it is pinned against the exact-rational model (tests/golden/, cases named ocp_*) and against a
 * nearest-value search over the eight e2m1 magnitudes.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off (see Makefile).
 */
#include "cq_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ floats */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float cqo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t cqo_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest, ties to even */
    return (uint16_t)(u >> 16);
}

float cqo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1fu) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        /* zero or subnormal: man * 2^-24, exact in f32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t cqo_f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); /* NaN */
    if (a >= 0x47800000u) {
        /* |f| >= 65536: infinity (65520 <= |f| < 65536 rounds up below) */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a < 0x38800000u) {
        /* below the smallest normal half (2^-14): subnormal or zero.
         * Adding 0.5f aligns the 10 subnormal bits at the bottom of the f32
         * significand; the f32 add itself performs the round-to-nearest-even. */
        float v = bits_f32(a) + 0.5f;
        return (uint16_t)(sign | (f32_bits(v) - 0x3f000000u));
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u); /* RNE on the 13 dropped bits */
    return (uint16_t)(sign | ((r - 0x38000000u) >> 13)); /* may carry into inf */
}

/* Generic small-float encoder: 1 sign, `ebits` exponent (bias `bias`), `mbits`
 * mantissa; round-to-nearest-even, subnormals kept, magnitudes above `maxval`
 * saturate to `maxcode` (finite).  NaN -> `nancode`. */
static uint8_t encode_minifloat(float f, int ebits, int mbits, int bias, float maxval,
                                uint8_t maxcode, uint8_t nancode) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 31) << (ebits + mbits));
    float a = fabsf(f);
    if (a != a) return (uint8_t)(sign | nancode);
    if (a >= maxval) return (uint8_t)(sign | maxcode);
    if (a == 0.0f) return sign;
    int e;
    (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) -> exponent of leading bit = e-1 */
    int lead = e - 1;
    int emin = 1 - bias; /* exponent of the smallest normal */
    if (lead < emin) lead = emin;
    /* quantum = 2^(lead - mbits); a / quantum is exact in f32 for these widths */
    float q = ldexpf(a, mbits - lead);
    float r = rintf(q); /* RNE under the default rounding mode */
    uint32_t ri = (uint32_t)r;
    uint32_t code;
    if (lead == emin && ri < (1u << mbits)) {
        code = ri; /* subnormal */
    } else {
        /* ri in [2^mbits, 2^(mbits+1)]; equality with the upper end = carry */
        uint32_t ex = (uint32_t)(lead + bias);
        if (ri == (2u << mbits)) {
            ex += 1;
            ri = 1u << mbits;
        }
        code = (ex << mbits) | (ri - (1u << mbits));
    }
    if (code > maxcode) code = maxcode;
    return (uint8_t)(sign | code);
}

static float decode_minifloat(uint8_t b, int ebits, int mbits, int bias) {
    uint32_t sign = (b >> (ebits + mbits)) & 1u;
    uint32_t ex = (b >> mbits) & ((1u << ebits) - 1u);
    uint32_t man = b & ((1u << mbits) - 1u);
    float v;
    if (ex == 0)
        v = ldexpf((float)man, 1 - bias - mbits);
    else
        v = ldexpf((float)(man | (1u << mbits)), (int)ex - bias - mbits);
    return sign ? -v : v;
}

/* OCP e4m3 (fn variant): bias 7, max 448 = 0x7e, NaN = 0x7f, no infinity. */
uint8_t cqo_f32_to_e4m3(float f) { return encode_minifloat(f, 4, 3, 7, 448.0f, 0x7e, 0x7f); }
float cqo_e4m3_to_f32(uint8_t b) {
    if ((b & 0x7f) == 0x7f) return bits_f32(0x7fc00000u);
    return decode_minifloat(b, 4, 3, 7);
}
/* e5m2: bias 15, max finite 57344 = 0x7b, inf = 0x7c, NaN = 0x7e. */
uint8_t cqo_f32_to_e5m2(float f) { return encode_minifloat(f, 5, 2, 15, 57344.0f, 0x7b, 0x7e); }
float cqo_e5m2_to_f32(uint8_t b) {
    if ((b & 0x7c) == 0x7c) {
        if (b & 3) return bits_f32(0x7fc00000u);
        return (b & 0x80) ? -INFINITY : INFINITY;
    }
    return decode_minifloat(b, 5, 2, 15);
}
/* OCP e2m1: bias 1, values {0,.5,1,1.5,2,3,4,6}; no NaN (mapped to +6 here, never reached). */
uint8_t cqo_f32_to_e2m1(float f) { return encode_minifloat(f, 2, 1, 1, 6.0f, 0x7, 0x7); }
float cqo_e2m1_to_f32(uint8_t n) { return decode_minifloat((uint8_t)(n & 0xf), 2, 1, 1); }

static inline float load_f(const void* p, int dtype, uint64_t i) {
    switch (dtype) {
        case CQ_F32: return ((const float*)p)[i];
        case CQ_F16: return cqo_f16_to_f32(((const uint16_t*)p)[i]);
        default: return cqo_bf16_to_f32(((const uint16_t*)p)[i]);
    }
}
static inline void store_f(void* p, int dtype, uint64_t i, float v) {
    switch (dtype) {
        case CQ_F32: ((float*)p)[i] = v; break;
        case CQ_F16: ((uint16_t*)p)[i] = cqo_f32_to_f16(v); break;
        default: ((uint16_t*)p)[i] = cqo_f32_to_bf16(v); break;
    }
}
/* round an f32 value to the precision of `dtype`, result widened back to f32 */
static inline float round_to(int dtype, float v) {
    switch (dtype) {
        case CQ_F32: return v;
        case CQ_F16: return cqo_f16_to_f32(cqo_f32_to_f16(v));
        default: return cqo_bf16_to_f32(cqo_f32_to_bf16(v));
    }
}
static inline int param_dtype(uint8_t param) {
    return param == CQ_PARAM_F32 ? CQ_F32 : (param == CQ_PARAM_F16 ? CQ_F16 : CQ_BF16);
}

/* ------------------------------------------------------------------ scheme */

uint32_t cqo_value_size_bits(uint8_t value) {
    switch (value) {
        case CQ_VALUE_Q8F: case CQ_VALUE_Q8S: case CQ_VALUE_E4M3: case CQ_VALUE_E5M2: return 8;
        case CQ_VALUE_Q4F: case CQ_VALUE_Q4S: case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: return 4;
        case CQ_VALUE_Q2F: case CQ_VALUE_Q2S: return 2;
        default: return 0;
    }
}

/* stored bits / value bits (call sites src/quantize.rs:144,290; the comment
 * "32 / 8 = 4" at src/quantize.rs:305; tests/suite/symmetric.rs:69).  For the
 * native store one stored element holds one value (two for E2M1 bytes). */
uint32_t cqo_num_quants(const cq_scheme* s) {
    uint32_t bits = cqo_value_size_bits(s->value);
    if (bits == 0) return 0;
    if (s->store == CQ_STORE_U32) return 32u / bits;
    return (s->value == CQ_VALUE_E2M1 || s->value == CQ_VALUE_E2M1_OCP) ? 2u : 1u;
}

int cqo_value_range(uint8_t value, float* lo, float* hi) {
    switch (value) {
        case CQ_VALUE_Q8F: *lo = -128.f; *hi = 127.f; return 0;
        case CQ_VALUE_Q8S: *lo = -127.f; *hi = 127.f; return 0;
        case CQ_VALUE_Q4F: *lo = -8.f; *hi = 7.f; return 0;
        case CQ_VALUE_Q4S: *lo = -7.f; *hi = 7.f; return 0;
        case CQ_VALUE_Q2F: *lo = -2.f; *hi = 1.f; return 0;
        case CQ_VALUE_Q2S: *lo = -1.f; *hi = 1.f; return 0;
        case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: *lo = -6.f; *hi = 6.f; return 0;
        case CQ_VALUE_E4M3: *lo = -448.f; *hi = 448.f; return 0;
        case CQ_VALUE_E5M2: *lo = -57344.f; *hi = 57344.f; return 0;
        default: return -1;
    }
}

/* block size of dimension d after left-padding the block vector with 1s
 * (BlockSize::to_dim_vec(rank), src/layout/scales.rs:239) */
static inline uint64_t block_dim(const cq_scheme* s, uint32_t rank, uint32_t d) {
    uint32_t pad = rank - s->block_rank;
    return d < pad ? 1u : s->block[d - pad];
}

/* ------------------------------------------------------------------ layout */

/* ScalesLayout::to_source_pos (src/layout/scales.rs:83-85 per-tensor,
 * :144-160 block-scaled): walk the dimensions last to first. */
uint64_t cqo_scale_index(const cq_scheme* s, uint32_t rank, const uint64_t* shape,
                         const uint64_t* scale_strides, uint64_t elem) {
    if (s->level == CQ_LEVEL_TENSOR) return 0;
    uint64_t offs = elem, scale_offs = 0;
    for (uint32_t i = 0; i < rank; i++) {
        uint32_t dim = rank - i - 1;
        uint64_t offs_local = offs % shape[dim];
        offs = offs / shape[dim];
        scale_offs += (offs_local / block_dim(s, rank, dim)) * scale_strides[dim];
    }
    return scale_offs;
}

/* ScalesLayout::is_block_start (src/layout/scales.rs:104-106, :179-194) */
int cqo_is_block_start(const cq_scheme* s, uint32_t rank, const uint64_t* shape, uint64_t elem) {
    if (s->level == CQ_LEVEL_TENSOR) return elem == 0;
    uint64_t offs = elem;
    int is_start = 1;
    for (uint32_t i = 0; i < rank; i++) {
        uint32_t dim = rank - i - 1;
        uint64_t offs_local = offs % shape[dim];
        offs = offs / shape[dim];
        is_start &= (offs_local % block_dim(s, rank, dim)) == 0;
    }
    return is_start;
}

/* ----------------------------------------------------------------- packing */

/* pack_q (src/quantize.rs:61-81): element i occupies bits [i*bits,(i+1)*bits),
 * two's-complement field. */
uint32_t cqo_pack_word(const int32_t* codes, uint32_t bits) {
    uint32_t nq = 32u / bits, mask = (1u << bits) - 1u, packed = 0;
    for (uint32_t i = 0; i < nq; i++) packed |= ((uint32_t)codes[i] & mask) << (i * bits);
    return packed;
}

/* unpack_q (src/dequantize.rs:86-118): raw - (raw >= 2^(bits-1)) * 2^bits */
void cqo_unpack_word(uint32_t word, uint32_t bits, int32_t* codes) {
    uint32_t nq = 32u / bits, mask = (1u << bits) - 1u, sign_bit = 1u << (bits - 1);
    int32_t two_pow_n = 1 << bits;
    for (uint32_t i = 0; i < nq; i++) {
        uint32_t raw = (word >> (i * bits)) & mask;
        int32_t is_negative = raw >= sign_bit;
        codes[i] = (int32_t)raw - is_negative * two_pow_n;
    }
}

/* quantize_symmetric (src/quantize.rs:19-31), one element, arithmetic in F */
static inline float quantize_one(float x, float d, int dtype, float lo, float hi) {
    float t = round_to(dtype, x / d); /* value / F(scale), true division */
    float r = rintf(t);               /* Line::round, exact in F */
    return fmaxf(lo, fminf(r, hi));   /* Line::clamp */
}

/* The extension value CQ_VALUE_E2M1_OCP (no counterpart in the reference): the quotient in F, clamped, WITHOUT the
 * integer rounding; the one rounding is the cast to e2m1 that follows (cqo_f32_to_e2m1: nearest, ties to even). */
static inline float quantize_one_unrounded(float x, float d, int dtype, float lo, float hi) {
    float t = round_to(dtype, x / d);
    return fmaxf(lo, fminf(t, hi));
}

/* write_scale (src/quantize.rs:83-98): FS(scale_in[idx]); store at block start.
 * Returns the divisor F(FS(scale)) widened to f32. */
static inline float write_scale(const cq_scheme* s, uint32_t rank, const uint64_t* shape,
                                const void* scale, const uint64_t* strides, void* out_scale,
                                const uint64_t* out_strides, int dtype, uint64_t elem) {
    int pd = param_dtype(s->param);
    uint64_t si = cqo_scale_index(s, rank, shape, strides, elem);
    float s_f = load_f(scale, dtype, si);
    float s_fs = round_to(pd, s_f);
    /* out_scale is a view of its own: same mapping, its own strides
     * (scales_view(.., out_scale, ..) at src/quantize.rs:317) */
    if (cqo_is_block_start(s, rank, shape, elem))
        store_f(out_scale, pd, cqo_scale_index(s, rank, shape, out_strides, elem), s_fs);
    return round_to(dtype, s_fs);
}

static uint64_t num_elements(uint32_t rank, const uint64_t* shape) {
    uint64_t n = 1;
    for (uint32_t i = 0; i < rank; i++) n *= shape[i];
    return n;
}

/* ------------------------------------------------------------- packed path */

/* quantize_symmetric_packed_kernel (src/quantize.rs:128-171), one word per step */
int cqo_quantize_packed(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                        const void* scale, const uint64_t* scale_strides, void* out_scale,
                        const uint64_t* out_scale_strides, uint32_t* output, const cq_scheme* s,
                        uint64_t word_begin, uint64_t word_end) {
    float lo, hi;
    if (s->store != CQ_STORE_U32 || cqo_value_range(s->value, &lo, &hi)) return -1;
    uint32_t bits = cqo_value_size_bits(s->value), nq = 32u / bits;
    for (uint64_t p = word_begin; p < word_end; p++) {
        uint64_t packed_pos = p * nq;
        float d = write_scale(s, rank, shape, scale, scale_strides, out_scale, out_scale_strides,
                              dtype, packed_pos);
        int32_t codes[16];
        for (uint32_t i = 0; i < nq; i++) {
            float x = load_f(input, dtype, packed_pos + i);
            codes[i] = s->value == CQ_VALUE_E2M1_OCP ? (int32_t)cqo_f32_to_e2m1(quantize_one_unrounded(x, d, dtype, lo, hi))
                                                      : (int32_t)quantize_one(x, d, dtype, lo, hi);
        }
        output[p] = cqo_pack_word(codes, bits);
    }
    return 0;
}

/* dequantize_symmetric_packed_kernel (src/dequantize.rs:120-148) with
 * dequantize_symmetric_packed_value (:60-79) and dequantize_symmetric (:22-25) */
int cqo_dequantize_packed(const uint32_t* values, uint32_t rank, const uint64_t* shape,
                          const void* params, const uint64_t* scale_strides, void* output,
                          int dtype, const cq_scheme* s, uint64_t word_begin, uint64_t word_end) {
    if (s->store != CQ_STORE_U32) return -1;
    uint32_t bits = cqo_value_size_bits(s->value);
    if (!bits) return -1;
    uint32_t nq = 32u / bits;
    int pd = param_dtype(s->param);
    for (uint64_t p = word_begin; p < word_end; p++) {
        uint64_t e0 = p * nq;
        uint64_t si = cqo_scale_index(s, rank, shape, scale_strides, e0);
        float sc = round_to(dtype, load_f(params, pd, si)); /* Line::cast_from(scale) */
        int32_t codes[16];
        cqo_unpack_word(values[p], bits, codes);
        for (uint32_t i = 0; i < nq; i++) {
            float v = (float)codes[i]; /* F::cast_from(signed_value), exact */
            if (s->value == CQ_VALUE_E2M1_OCP) v = cqo_e2m1_to_f32((uint8_t)(codes[i] & 0xf)); /* extension: the nibble decoded */
            store_f(output, dtype, e0 + i, sc * v);
        }
    }
    return 0;
}

/* ------------------------------------------------------------- native path */

/* quantize_symmetric_native_kernel (src/quantize.rs:100-126) */
int cqo_quantize_native(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                        const void* scale, const uint64_t* scale_strides, void* out_scale,
                        const uint64_t* out_scale_strides, uint8_t* output, const cq_scheme* s,
                        uint64_t elem_begin, uint64_t elem_end) {
    float lo, hi;
    if (s->store != CQ_STORE_NATIVE || cqo_value_range(s->value, &lo, &hi)) return -1;
    for (uint64_t e = elem_begin; e < elem_end; e++) {
        float d = write_scale(s, rank, shape, scale, scale_strides, out_scale, out_scale_strides,
                              dtype, e);
        float c = s->value == CQ_VALUE_E2M1_OCP ? quantize_one_unrounded(load_f(input, dtype, e), d, dtype, lo, hi)
                                                : quantize_one(load_f(input, dtype, e), d, dtype, lo, hi);
        switch (s->value) {
            case CQ_VALUE_Q8F: case CQ_VALUE_Q8S: output[e] = (uint8_t)(int8_t)(int32_t)c; break;
            case CQ_VALUE_E4M3: output[e] = cqo_f32_to_e4m3(c); break;
            case CQ_VALUE_E5M2: output[e] = cqo_f32_to_e5m2(c); break;
            case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: {
                uint8_t nib = cqo_f32_to_e2m1(c);
                uint8_t old = (e & 1) ? output[e >> 1] : 0;
                output[e >> 1] = (e & 1) ? (uint8_t)((old & 0x0f) | (nib << 4)) : nib;
                break;
            }
            default: return -1;
        }
    }
    return 0;
}

/* dequantize_symmetric_native_kernel (src/dequantize.rs:150-167) */
int cqo_dequantize_native(const uint8_t* values, uint32_t rank, const uint64_t* shape,
                          const void* params, const uint64_t* scale_strides, void* output,
                          int dtype, const cq_scheme* s, uint64_t elem_begin, uint64_t elem_end) {
    if (s->store != CQ_STORE_NATIVE) return -1;
    int pd = param_dtype(s->param);
    for (uint64_t e = elem_begin; e < elem_end; e++) {
        uint64_t si = cqo_scale_index(s, rank, shape, scale_strides, e);
        float sc = round_to(dtype, load_f(params, pd, si));
        float v;
        switch (s->value) {
            case CQ_VALUE_Q8F: case CQ_VALUE_Q8S: v = (float)(int8_t)values[e]; break;
            case CQ_VALUE_E4M3: v = cqo_e4m3_to_f32(values[e]); break;
            case CQ_VALUE_E5M2: v = cqo_e5m2_to_f32(values[e]); break;
            case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: v = cqo_e2m1_to_f32((values[e >> 1] >> ((e & 1) * 4)) & 0xf); break;
            default: return -1;
        }
        store_f(output, dtype, e, sc * round_to(dtype, v));
    }
    return 0;
}

/* ------------------------------------------------------------------ scales */

/* Scale rule of the reference's tests (tests/suite/symmetric.rs:35-38 per
 * tensor, :156-179 per block): 2*max(|min|,|max|) / (q_max - q_min) in f32.
 * max|x| over a block equals max(|min|,|max|); NaN elements are ignored the way
 * Rust's f32::max/min ignore them.  Blocks are N-D boxes (src/layout/scales.rs). */
int cqo_compute_scales(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                       void* scales, const cq_scheme* s) {
    float lo, hi;
    if (cqo_value_range(s->value, &lo, &hi)) return -1;
    uint64_t n = num_elements(rank, shape);
    uint64_t sshape[CQ_MAX_RANK], sstrides[CQ_MAX_RANK], ns = 1;
    if (s->level == CQ_LEVEL_TENSOR) {
        ns = 1;
    } else {
        for (uint32_t d = 0; d < rank; d++) {
            uint64_t b = block_dim(s, rank, d);
            sshape[d] = (shape[d] + b - 1) / b;
        }
        for (int d = (int)rank - 1; d >= 0; d--) {
            sstrides[d] = ns;
            ns *= sshape[d];
        }
    }
    float* amax = (float*)calloc(ns, sizeof(float));
    if (!amax) return -2;
    for (uint64_t e = 0; e < n; e++) {
        uint64_t si = cqo_scale_index(s, rank, shape, sstrides, e);
        float a = fabsf(load_f(input, dtype, e));
        amax[si] = fmaxf(amax[si], a); /* fmaxf drops NaN */
    }
    for (uint64_t i = 0; i < ns; i++) {
        float range = 2.0f * amax[i];
        store_f(scales, dtype, i, range / (hi - lo));
    }
    free(amax);
    return 0;
}

/* MaxAbs along one axis (crates/cubek-reduce/src/instructions/maxabs.rs:47-96:
 * identity 0, keep the larger of accumulator and |item|); NaN items are ignored.
 * Any strides; output has extent 1 on `axis`. */
int cqo_reduce_max_abs(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                       const uint64_t* in_strides, uint32_t axis, void* output,
                       const uint64_t* out_strides) {
    if (axis >= rank) return -1;
    uint64_t num_out = 1;
    for (uint32_t d = 0; d < rank; d++)
        if (d != axis) num_out *= shape[d];
    for (uint64_t i = 0; i < num_out; i++) {
        uint64_t rem = i, in_off = 0, out_off = 0;
        for (int d = (int)rank - 1; d >= 0; d--) {
            if ((uint32_t)d == axis) continue;
            uint64_t c = rem % shape[d];
            rem /= shape[d];
            in_off += c * in_strides[d];
            out_off += c * out_strides[d];
        }
        float m = 0.0f;
        for (uint64_t k = 0; k < shape[axis]; k++)
            m = fmaxf(m, fabsf(load_f(input, dtype, in_off + k * in_strides[axis])));
        store_f(output, dtype, out_off, m);
    }
    return 0;
}

/* Re-pack a strided quantized tensor into a contiguous one packed along the last
 * dimension: what cubek-matmul asks of cubecl-std's into_contiguous_packed
 * (crates/cubek-matmul/src/base.rs:505-529).  `shape` is the logical (unpacked)
 * shape; the input stores `packing` values per element along `packed_dim`, value 0
 * in the low bits, and is addressed through `in_strides`; output element `pos`
 * gathers the logical values pos*packing .. pos*packing+packing-1.
 * parity unpinned: cubecl-std is not vendored with the reference. */
int cqo_into_contiguous_packed(const void* input, uint32_t elem_bytes, uint32_t packing, uint32_t rank,
                               const uint64_t* shape, const uint64_t* in_strides, uint32_t packed_dim,
                               void* output) {
    if ((elem_bytes != 1 && elem_bytes != 4) || packing == 0 || (8 * elem_bytes) % packing || rank == 0 ||
        packed_dim >= rank || shape[rank - 1] % packing || shape[packed_dim] % packing)
        return -1;
    const uint32_t bits = 8 * elem_bytes / packing;
    const uint32_t mask = bits == 32 ? 0xffffffffu : (1u << bits) - 1u;
    uint64_t n = 1;
    for (uint32_t d = 0; d < rank; d++) n *= shape[d];
    for (uint64_t pos = 0; pos < n / packing; pos++) {
        uint32_t out = 0;
        for (uint32_t k = 0; k < packing; k++) {
            uint64_t rem = pos * packing + k, off = 0, sub = 0;
            for (int d = (int)rank - 1; d >= 0; d--) {
                uint64_t c = rem % shape[d];
                rem /= shape[d];
                if ((uint32_t)d == packed_dim) {
                    sub = c % packing;
                    c /= packing;
                }
                off += c * in_strides[d];
            }
            uint32_t word = elem_bytes == 4 ? ((const uint32_t*)input)[off] : ((const uint8_t*)input)[off];
            out |= ((word >> (sub * bits)) & mask) << (k * bits);
        }
        if (elem_bytes == 4)
            ((uint32_t*)output)[pos] = out;
        else
            ((uint8_t*)output)[pos] = (uint8_t)out;
    }
    return 0;
}

/* --------------------------------------------------------- threaded drivers */

typedef struct {
    int kind; /* 0 quantize, 1 dequantize */
    const void* a;
    int dtype;
    uint32_t rank;
    const uint64_t* shape;
    const void* scale;
    const uint64_t* strides;
    void* out_scale;
    const uint64_t* out_strides;
    void* out;
    const cq_scheme* s;
    uint64_t wb, we;
    int rc;
} job_t;

static void* run_job(void* arg) {
    job_t* j = (job_t*)arg;
    if (j->kind == 0)
        j->rc = cqo_quantize_packed(j->a, j->dtype, j->rank, j->shape, j->scale, j->strides,
                                    j->out_scale, j->out_strides, (uint32_t*)j->out, j->s, j->wb,
                                    j->we);
    else
        j->rc = cqo_dequantize_packed((const uint32_t*)j->a, j->rank, j->shape, j->scale,
                                      j->strides, j->out, j->dtype, j->s, j->wb, j->we);
    return NULL;
}

static int run_mt(job_t base, int threads) {
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    pthread_t tid[256];
    job_t jobs[256];
    uint64_t total = base.we - base.wb;
    /* split on multiples of 64 words so that no two threads share a block start */
    uint64_t per = ((total + (uint64_t)threads - 1) / (uint64_t)threads + 63) / 64 * 64;
    int used = 0;
    for (int t = 0; t < threads; t++) {
        uint64_t b = base.wb + per * (uint64_t)t;
        if (b >= base.we) break;
        uint64_t e = b + per < base.we ? b + per : base.we;
        jobs[t] = base;
        jobs[t].wb = b;
        jobs[t].we = e;
        pthread_create(&tid[t], NULL, run_job, &jobs[t]);
        used++;
    }
    int rc = 0;
    for (int t = 0; t < used; t++) {
        pthread_join(tid[t], NULL);
        if (jobs[t].rc) rc = jobs[t].rc;
    }
    return rc;
}

int cqo_quantize_packed_mt(const void* input, int dtype, uint32_t rank, const uint64_t* shape,
                           const void* scale, const uint64_t* scale_strides, void* out_scale,
                           const uint64_t* out_scale_strides, uint32_t* output, const cq_scheme* s,
                           uint64_t word_begin, uint64_t word_end, int threads) {
    job_t j = {0, input, dtype, rank, shape, scale, scale_strides, out_scale, out_scale_strides,
               output, s, word_begin, word_end, 0};
    return run_mt(j, threads);
}

int cqo_dequantize_packed_mt(const uint32_t* values, uint32_t rank, const uint64_t* shape,
                             const void* params, const uint64_t* scale_strides, void* output,
                             int dtype, const cq_scheme* s, uint64_t word_begin,
                             uint64_t word_end, int threads) {
    job_t j = {1, values, dtype, rank, shape, params, scale_strides, NULL, NULL, output, s,
               word_begin, word_end, 0};
    return run_mt(j, threads);
}
