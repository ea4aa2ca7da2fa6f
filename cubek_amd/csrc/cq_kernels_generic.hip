// Generic quantize / dequantize kernels: any rank, any strides, N-D blocks, strided
// scale tensors, ragged tails, native (byte) store.  One thread per stored element,
// scale addressing exactly as the reference's BlockScaledLayout
// (crates/cubek-quant/src/layout/scales.rs:144-160, :179-194).  These kernels
// are the fallback and tail path; the streaming shapes take the flat kernels.
#include "cq_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;

struct ScalePos {
    uint64_t a, b;  // offsets into scale_in / scale_out
    bool start;     // first element of its block
};

// to_source_pos + is_block_start in one walk over the dimensions, last to first.
__device__ __forceinline__ ScalePos scale_pos(const Layout& L, uint64_t elem) {
    ScalePos r{0, 0, true};
    if (L.rank == 0) {
        r.start = elem == 0;
        return r;
    }
    uint64_t offs = elem;
    for (int d = static_cast<int>(L.rank) - 1; d >= 0; d--) {
        uint32_t local = static_cast<uint32_t>(offs % L.shape[d]);
        offs /= L.shape[d];
        uint32_t blk = local / L.block[d];
        r.a += static_cast<uint64_t>(blk) * L.stride_a[d];
        r.b += static_cast<uint64_t>(blk) * L.stride_b[d];
        r.start = r.start && (local % L.block[d] == 0);
    }
    return r;
}

// Memory offsets of stored element `p` (logical, row-major over the packed shape) and
// of the first of its `per` float elements; `step` is the float tensor's stride along
// the last dimension.
struct ValuePos {
    uint64_t f, v, step;
};

__device__ __forceinline__ ValuePos value_pos(const ValueStrides& S, uint64_t p, uint32_t per) {
    if (!S.on) return ValuePos{p * per, p, 1};
    const int last = static_cast<int>(S.rank) - 1;
    ValuePos r{0, 0, S.floats[last]};
    uint64_t rem = p;
    for (int d = last; d >= 0; d--) {
        const uint32_t n = d == last ? S.shape[d] / per : S.shape[d];
        const uint64_t c = rem % n;
        rem /= n;
        r.f += c * (d == last ? per : 1u) * S.floats[d];
        r.v += c * S.stored[d];
    }
    return r;
}

// write_scale (src/quantize.rs:83-98); returns the divisor F(FS(scale)).
template <class F>
__device__ __forceinline__ float fetch_divisor(const GenericArgs& a, uint64_t elem) {
    ScalePos sp = scale_pos(a.layout, elem);
    float s_f = load_dtype(a.scale_in_dtype, a.scale_in, sp.a);
    float s_fs = round_to_dtype(a.param_dtype, s_f);
    if (a.scale_out != nullptr && sp.start) store_dtype(a.param_dtype, a.scale_out, sp.b, s_fs);
    return F::round(s_fs);
}

__device__ __forceinline__ float decode_native(int value, uint32_t b);

// The extension value CQ_VALUE_E2M1_OCP: the clamped quotient in F, cast once to e2m1 (nearest, ties to the even code;
// the sign bit is the float's).
template <class F>
__device__ __forceinline__ uint32_t quantize_e2m1_unrounded(float x, float d, float lo, float hi) {
    const float c = clamp_code(F::round(x / d), lo, hi);
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, c, 0.0f, 1.0f, 0) & 0xfu;
}

template <class F>
__global__ __launch_bounds__(kThreads) void quantize_generic_kernel(GenericArgs a, int bits) {
    uint64_t p = a.word_begin + static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (p >= a.word_end) return;
    const uint32_t nq = 32u / bits, mask = (1u << bits) - 1u;
    const uint64_t e0 = p * nq;
    const float d = fetch_divisor<F>(a, e0);
    const ValuePos vp = value_pos(a.vs, p, nq);
    uint32_t w = 0;
    for (uint32_t i = 0; i < nq; i++) {
        const float x = F::load(a.input, vp.f + i * vp.step);
        if (a.value == CQ_VALUE_E2M1_OCP) {
            w |= quantize_e2m1_unrounded<F>(x, d, a.range.lo, a.range.hi) << (i * bits);
            continue;
        }
        float q = quantize_exact<F>(x, d, a.range.lo, a.range.hi);
        w |= (static_cast<uint32_t>(static_cast<int32_t>(q)) & mask) << (i * bits);
    }
    static_cast<uint32_t*>(a.output)[vp.v] = w;
}

template <class F>
__global__ __launch_bounds__(kThreads) void dequantize_generic_kernel(GenericArgs a, int bits) {
    uint64_t p = a.word_begin + static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (p >= a.word_end) return;
    const uint32_t nq = 32u / bits;
    const uint64_t e0 = p * nq;
    ScalePos sp = scale_pos(a.layout, e0);
    const float s = F::round(load_dtype(a.param_dtype, a.scale_in, sp.a));
    const ValuePos vp = value_pos(a.vs, p, nq);
    const uint32_t w = static_cast<const uint32_t*>(a.input)[vp.v];
    for (uint32_t i = 0; i < nq; i++) {
        int32_t v = static_cast<int32_t>(w << (32 - bits - i * bits)) >> (32 - bits);
        const float q = a.value == CQ_VALUE_E2M1_OCP ? decode_native(CQ_VALUE_E2M1, (w >> (i * bits)) & 0xfu) : static_cast<float>(v);
        F::store(a.output, vp.f + i * vp.step, s * q);
    }
}

// One thread per block: abs-max over the block's N-D box.
template <class F>
__global__ __launch_bounds__(kThreads) void scales_generic_kernel(GenericArgs a, int out_dtype,
                                                                  uint64_t num_blocks) {
    uint64_t b = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (b >= num_blocks) return;
    const Layout& L = a.layout;
    // block coordinates (row-major over shape/block) and the box origin
    uint32_t origin[CQ_MAX_RANK];
    uint64_t out_off = 0, rem = b, volume = 1;
    for (int d = static_cast<int>(L.rank) - 1; d >= 0; d--) {
        uint32_t nb = L.shape[d] / L.block[d];
        uint32_t bc = static_cast<uint32_t>(rem % nb);
        rem /= nb;
        origin[d] = bc * L.block[d];
        out_off += static_cast<uint64_t>(bc) * L.stride_b[d];
        volume *= L.block[d];
    }
    float amax = 0.0f;
    for (uint64_t k = 0; k < volume; k++) {
        uint64_t kr = k, lin = 0, mul = 1;
        for (int d = static_cast<int>(L.rank) - 1; d >= 0; d--) {
            uint32_t o = static_cast<uint32_t>(kr % L.block[d]);
            kr /= L.block[d];
            lin += static_cast<uint64_t>(origin[d] + o) * (a.vs.on ? a.vs.floats[d] : mul);
            mul *= L.shape[d];
        }
        amax = fmaxf(amax, fabsf(F::load(a.input, lin)));
    }
    float s_f = F::round(scale_from_absmax(amax, a.range.hi - a.range.lo));
    store_dtype(out_dtype, a.scale_out, out_off, round_to_dtype(out_dtype, s_f));
}

// ---- native store ----------------------------------------------------------

__device__ __forceinline__ uint32_t encode_native(int value, float c) {
    switch (value) {
        case CQ_VALUE_E4M3:
            return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(c, 0.0f, 0, false)) & 0xffu;
        case CQ_VALUE_E5M2:
            return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_bf8_f32(c, 0.0f, 0, false)) & 0xffu;
        case CQ_VALUE_E2M1: {
            // c is an integer in [-6,6]: 0,1,2,3,4,6 are e2m1 values, 5 ties to 4 (even
            // mantissa); the sign bit is the float's, so -0.0 stays -0 as in a float cast
            uint32_t m = static_cast<uint32_t>(static_cast<int32_t>(fabsf(c)));
            return ((0x7665420u >> (4 * m)) & 0x7u) | ((f32_bits(c) >> 28) & 0x8u);
        }
        default:
            return static_cast<uint32_t>(static_cast<int32_t>(c)) & 0xffu;  // i8
    }
}

__device__ __forceinline__ float decode_native(int value, uint32_t b) {
    switch (value) {
        case CQ_VALUE_E4M3: return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(b), 0);
        case CQ_VALUE_E5M2: return __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(b), 0);
        case CQ_VALUE_E2M1: case CQ_VALUE_E2M1_OCP: {
            uint32_t m = b & 7u;
            uint32_t bits = m == 0 ? 0u : (m == 1 ? 0x3f000000u : (((m >> 1) + 126u) << 23) | ((m & 1u) << 22));
            return bits_f32(bits | ((b & 8u) << 28));
        }
        default: return static_cast<float>(static_cast<int8_t>(b));
    }
}

// quantize_symmetric_native_kernel (src/quantize.rs:100-126), one thread per stored byte
template <class F>
__global__ __launch_bounds__(kThreads) void quantize_native_kernel(GenericArgs a) {
    uint64_t j = a.word_begin + static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (j >= a.word_end) return;
    uint8_t* out = static_cast<uint8_t*>(a.output);
    if (a.value == CQ_VALUE_E2M1 || a.value == CQ_VALUE_E2M1_OCP) {
        const ValuePos vp = value_pos(a.vs, j, 2);
        uint32_t byte = 0;
        for (uint32_t h = 0; h < 2; h++) {
            float d = fetch_divisor<F>(a, 2 * j + h);
            const float x = F::load(a.input, vp.f + h * vp.step);
            if (a.value == CQ_VALUE_E2M1_OCP) {
                byte |= quantize_e2m1_unrounded<F>(x, d, a.range.lo, a.range.hi) << (4 * h);
                continue;
            }
            float c = quantize_exact<F>(x, d, a.range.lo, a.range.hi);
            byte |= encode_native(a.value, c) << (4 * h);
        }
        out[vp.v] = static_cast<uint8_t>(byte);
    } else {
        const ValuePos vp = value_pos(a.vs, j, 1);
        float d = fetch_divisor<F>(a, j);
        float c = quantize_exact<F>(F::load(a.input, vp.f), d, a.range.lo, a.range.hi);
        out[vp.v] = static_cast<uint8_t>(encode_native(a.value, c));
    }
}

// dequantize_symmetric_native_kernel (src/dequantize.rs:150-167)
template <class F>
__global__ __launch_bounds__(kThreads) void dequantize_native_kernel(GenericArgs a) {
    uint64_t j = a.word_begin + static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (j >= a.word_end) return;
    const uint32_t per = (a.value == CQ_VALUE_E2M1 || a.value == CQ_VALUE_E2M1_OCP) ? 2u : 1u;
    const ValuePos vp = value_pos(a.vs, j, per);
    const uint8_t b = static_cast<const uint8_t*>(a.input)[vp.v];
    for (uint32_t h = 0; h < per; h++) {
        ScalePos sp = scale_pos(a.layout, per * j + h);
        float s = F::round(load_dtype(a.param_dtype, a.scale_in, sp.a));
        float v = decode_native(a.value, per == 2 ? (b >> (4 * h)) & 0xfu : b);
        F::store(a.output, vp.f + h * vp.step, s * F::round(v));
    }
}

// Per-tensor abs-max of a strided float tensor, pass 1: grid-stride over the logical
// elements, one f32 partial per workgroup.
template <class F>
__global__ __launch_bounds__(kThreads) void absmax_partials_strided_kernel(GenericArgs a, uint64_t num_elems,
                                                                           float* __restrict__ partials) {
    float m = 0.0f;
    for (uint64_t e = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x; e < num_elems;
         e += static_cast<uint64_t>(gridDim.x) * kThreads)
        m = fmaxf(m, fabsf(F::load(a.input, value_pos(a.vs, e, 1).f)));
    m = group_max<kWave>(m);
    __shared__ float lds[kThreads / kWave];
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kThreads / kWave; w++) m = fmaxf(m, lds[w]);
        partials[blockIdx.x] = m;
    }
}

inline dim3 grid_for(uint64_t n) { return dim3(static_cast<uint32_t>((n + kThreads - 1) / kThreads)); }

#define CQ_SWITCH_DTYPE(D, ...)                          \
    switch (D) {                                         \
        case CQ_F32: { using kF = F32; __VA_ARGS__; }    \
        case CQ_BF16: { using kF = BF16; __VA_ARGS__; }  \
        case CQ_F16: { using kF = F16; __VA_ARGS__; }    \
        default: return hipErrorInvalidValue;            \
    }

}  // namespace

hipError_t launch_quantize_generic(hipStream_t s, int dtype, int bits, const GenericArgs& a) {
    if (a.word_end <= a.word_begin) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((quantize_generic_kernel<kF>), grid_for(a.word_end - a.word_begin),
                                              dim3(kThreads), 0, s, a, bits);
                    return hipGetLastError())
}

hipError_t launch_dequantize_generic(hipStream_t s, int dtype, int bits, const GenericArgs& a) {
    if (a.word_end <= a.word_begin) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((dequantize_generic_kernel<kF>), grid_for(a.word_end - a.word_begin),
                                              dim3(kThreads), 0, s, a, bits);
                    return hipGetLastError())
}

hipError_t launch_scales_generic(hipStream_t s, int dtype, int out_dtype, const GenericArgs& a,
                                 uint64_t num_blocks) {
    if (num_blocks == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((scales_generic_kernel<kF>), grid_for(num_blocks), dim3(kThreads), 0, s,
                                              a, out_dtype, num_blocks);
                    return hipGetLastError())
}

hipError_t launch_absmax_partials_strided(hipStream_t s, int dtype, const GenericArgs& a, uint64_t num_elems,
                                          float* partials, uint32_t* num_partials) {
    const uint64_t want = (num_elems + kThreads * 8 - 1) / (kThreads * 8);
    const uint32_t grid = static_cast<uint32_t>(want < 1 ? 1 : (want > kMaxPartials ? kMaxPartials : want));
    *num_partials = grid;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((absmax_partials_strided_kernel<kF>), dim3(grid), dim3(kThreads), 0, s, a,
                                              num_elems, partials);
                    return hipGetLastError())
}

hipError_t launch_quantize_native(hipStream_t s, int dtype, const GenericArgs& a) {
    if (a.word_end <= a.word_begin) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((quantize_native_kernel<kF>), grid_for(a.word_end - a.word_begin),
                                              dim3(kThreads), 0, s, a);
                    return hipGetLastError())
}

hipError_t launch_dequantize_native(hipStream_t s, int dtype, const GenericArgs& a) {
    if (a.word_end <= a.word_begin) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((dequantize_native_kernel<kF>), grid_for(a.word_end - a.word_begin),
                                              dim3(kThreads), 0, s, a);
                    return hipGetLastError())
}

}  // namespace cq
