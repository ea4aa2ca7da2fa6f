// Flat (contiguous) quantize / dequantize kernels for gfx950.
//
// Work decomposition.  The float tensor is cut into 16-byte chunks (8 bf16/f16
// or 4 f32 values).  Lane l of a 256-lane workgroup owns chunk
// (blockIdx*kUnroll + u)*256 + l for u = 0..kUnroll-1, so every
// global_load_dwordx4 / global_store_dwordx4 instruction of a wave covers one
// contiguous 1 KiB segment.  A quantization block of B elements spans
// kGroup = B / values-per-chunk adjacent lanes (a power of two inside one wave):
// its abs-max is a DPP butterfly, no LDS.  Codes narrower than a word
// (chunk bits 16 or 8) are OR-combined across 2 or 4 lanes before one store.
//
// HBM traffic per element is the algorithmic minimum: the input once, the
// codes once, one scale per block.  Loads and stores carry the non-temporal
// hint: nothing is re-read.
#include "cq_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;

// kParamF32: the stored scales are f32 (the common case, resolved at compile
// time); otherwise `param_dtype_rt` selects f16 / bf16 at run time.
template <class F, int kBits, int kGroup, bool kDynamic, bool kParamF32, int kUnroll>
__global__ __launch_bounds__(kThreads) void quantize_flat_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    int scale_in_dtype, void* __restrict__ scale_out, int param_dtype_rt, uint64_t num_chunks,
    float lo, float hi) {
    const int param_dtype = kParamF32 ? static_cast<int>(CQ_F32) : param_dtype_rt;
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;  // 64, 32, 16 or 8
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;

    // Out-of-range lanes re-read the last chunk instead of branching, so all
    // kUnroll loads are issued back to back; only their stores are masked.
    const uint64_t last = num_chunks - 1;
    u32x4 raw[kUnroll];
    float s_given[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        c = c < num_chunks ? c : last;
        raw[u] = __builtin_nontemporal_load(in + c);
        if constexpr (!kDynamic)
            s_given[u] = load_dtype(scale_in_dtype, scale_in, kGroup == 0 ? 0 : c / (kGroup == 0 ? 1 : kGroup));
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic

#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        const bool live = c < num_chunks;
        float v[kN];
        F::unpack(raw[u], v);

        const uint64_t si = kGroup == 0 ? 0 : c / (kGroup == 0 ? 1 : kGroup);
        float s_f;
        if constexpr (kDynamic) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
            amax = group_max<kGroup>(amax);
            s_f = F::round(scale_from_absmax(amax, hi - lo));
        } else {
            s_f = s_given[u];
        }
        // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first lane
        const float s_fs = round_to_dtype(param_dtype, s_f);
        const bool block_start = kGroup == 0 ? c == 0 : (c % (kGroup == 0 ? 1 : kGroup)) == 0;
        if (scale_out != nullptr && live && block_start) store_dtype(param_dtype, scale_out, si, s_fs);
        const float d = F::round(s_fs);

        float q[kN];
        quantize_values<F, kN>(v, d, lo, hi, q);

        if constexpr (kChunkBits == 64) {
            u32x2 w = {pack_fields<kBits, 4>(q), pack_fields<kBits, 4>(q + 4)};
            if (live) __builtin_nontemporal_store(w, reinterpret_cast<u32x2*>(out) + c);
        } else if constexpr (kChunkBits == 32) {
            uint32_t w = pack_fields<kBits, kN>(q);
            if (live) __builtin_nontemporal_store(w, out + c);
        } else {
            constexpr int kLanesPerWord = 32 / kChunkBits;  // 2 or 4
            const uint32_t sub = static_cast<uint32_t>(c) & (kLanesPerWord - 1);
            uint32_t w = group_or<kLanesPerWord>(pack_fields<kBits, kN>(q) << (sub * kChunkBits));
            if (live && sub == 0) __builtin_nontemporal_store(w, out + c / kLanesPerWord);
        }
    }
}

template <class F, int kBits, int kGroup, bool kParamF32, int kUnroll>
__global__ __launch_bounds__(kThreads) void dequantize_flat_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params,
    int param_dtype_rt, uint64_t num_chunks) {
    const int param_dtype = kParamF32 ? static_cast<int>(CQ_F32) : param_dtype_rt;
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;

    const uint64_t last = num_chunks - 1;
    uint32_t w0[kUnroll], w1[kUnroll];
    float sc[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        c = c < num_chunks ? c : last;  // clamp instead of branching; stores are masked below
        w1[u] = 0;
        if constexpr (kChunkBits == 64) {
            u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(in) + c);
            w0[u] = w[0];
            w1[u] = w[1];
        } else if constexpr (kChunkBits == 32) {
            w0[u] = __builtin_nontemporal_load(in + c);
        } else {
            constexpr int kLanesPerWord = 32 / kChunkBits;
            uint32_t w = in[c / kLanesPerWord];  // neighbouring lanes share the word
            w0[u] = w >> ((static_cast<uint32_t>(c) & (kLanesPerWord - 1)) * kChunkBits);
        }
        const uint64_t si = kGroup == 0 ? 0 : c / (kGroup == 0 ? 1 : kGroup);
        sc[u] = F::round(load_dtype(param_dtype, params, si));  // Line::cast_from(scale)
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float y[kN];
        if constexpr (kChunkBits == 64) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                y[i] = sc[u] * unpack_field<kBits>(w0[u], i);
                y[i + 4] = sc[u] * unpack_field<kBits>(w1[u], i);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kN; i++) y[i] = sc[u] * unpack_field<kBits>(w0[u], i);
        }
        if (c < num_chunks) __builtin_nontemporal_store(F::pack(y), out + c);  // pack rounds to F
    }
}

// Block abs-max -> scale typed like the input (what quantize takes as `scale`).
template <class F, int kGroup, int kUnroll>
__global__ __launch_bounds__(kThreads) void scales_flat_kernel(const u32x4* __restrict__ in,
                                                               void* __restrict__ scales,
                                                               uint64_t num_chunks, float width) {
    constexpr int kN = F::kPerChunk;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
    const uint64_t last = num_chunks - 1;
    u32x4 raw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        raw[u] = __builtin_nontemporal_load(in + (c < num_chunks ? c : last));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float v[kN];
        F::unpack(raw[u], v);
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
        amax = group_max<kGroup>(amax);
        if (c < num_chunks && (c % kGroup) == 0)
            F::store(scales, c / kGroup, scale_from_absmax(amax, width));
    }
}

// Per-tensor abs-max, pass 1: grid-stride over chunks, one partial per workgroup.
template <class F>
__global__ __launch_bounds__(kThreads) void absmax_partials_kernel(const void* __restrict__ input,
                                                                   uint64_t num_elems,
                                                                   float* __restrict__ partials) {
    constexpr int kN = F::kPerChunk;
    const u32x4* in = static_cast<const u32x4*>(input);
    const uint64_t num_chunks = num_elems / kN;
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kThreads;
    float amax = 0.0f;
    for (uint64_t c = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x; c < num_chunks;
         c += stride) {
        float v[kN];
        F::unpack(in[c], v);
#pragma unroll
        for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {  // ragged tail, fewer than one chunk
        for (uint64_t e = num_chunks * kN; e < num_elems; e++)
            amax = fmaxf(amax, fabsf(F::load(input, e)));
    }
    amax = group_max<64>(amax);
    __shared__ float wave_max[kThreads / kWave];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = wave_max[0];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; w++) m = fmaxf(m, wave_max[w]);
        partials[blockIdx.x] = m;
    }
}

// Per-tensor scale from the partials: value = via(F(2*absmax/width)) stored as `out_dtype`.
__global__ __launch_bounds__(kThreads) void tensor_scale_kernel(const float* __restrict__ partials,
                                                                uint32_t num_partials, float width,
                                                                int f_dtype, int out_dtype,
                                                                void* __restrict__ out) {
    float amax = 0.0f;
    for (uint32_t i = threadIdx.x; i < num_partials; i += kThreads) amax = fmaxf(amax, partials[i]);
    amax = group_max<64>(amax);
    __shared__ float wave_max[kThreads / kWave];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = wave_max[0];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; w++) m = fmaxf(m, wave_max[w]);
        float s_f = round_to_dtype(f_dtype, scale_from_absmax(m, width));
        store_dtype(out_dtype, out, 0, round_to_dtype(out_dtype, s_f));
    }
}

inline uint32_t grid_for(uint64_t num_chunks, int unroll) {
    uint64_t per = static_cast<uint64_t>(kThreads) * unroll;
    return static_cast<uint32_t>((num_chunks + per - 1) / per);
}

int group_of(int dtype, uint32_t block) {
    if (block == 0) return 0;
    uint32_t per_chunk = dtype == CQ_F32 ? 4u : 8u;
    if (block % per_chunk) return -1;
    uint32_t g = block / per_chunk;
    if (g & (g - 1)) return -1;
    return g <= 32 ? static_cast<int>(g) : -1;
}

constexpr int kUnrollQ = 4;
constexpr int kUnrollD = 4;

template <class F, int kBits, int kGroup>
hipError_t quantize_launch(hipStream_t s, ScaleSource src, const FlatArgs& a) {
    dim3 grid(grid_for(a.num_chunks, kUnrollQ)), block(kThreads);
    auto in = static_cast<const u32x4*>(a.input);
    auto out = static_cast<uint32_t*>(a.output);
    const bool p32 = a.param_dtype == CQ_F32;
    if (src == ScaleSource::Dynamic) {
        if constexpr (kGroup > 0) {
            auto kernel = p32 ? quantize_flat_kernel<F, kBits, kGroup, true, true, kUnrollQ>
                              : quantize_flat_kernel<F, kBits, kGroup, true, false, kUnrollQ>;
            hipLaunchKernelGGL(kernel, grid, block, 0, s, in, out, nullptr, 0, a.scale_out,
                               a.param_dtype, a.num_chunks, a.range.lo, a.range.hi);
        } else {
            return hipErrorInvalidValue;
        }
    } else {
        auto kernel = p32 ? quantize_flat_kernel<F, kBits, kGroup, false, true, kUnrollQ>
                          : quantize_flat_kernel<F, kBits, kGroup, false, false, kUnrollQ>;
        hipLaunchKernelGGL(kernel, grid, block, 0, s, in, out, a.scale_in, a.scale_in_dtype,
                           a.scale_out, a.param_dtype, a.num_chunks, a.range.lo, a.range.hi);
    }
    return hipGetLastError();
}

template <class F, int kBits, int kGroup>
hipError_t dequantize_launch(hipStream_t s, const FlatArgs& a) {
    dim3 grid(grid_for(a.num_chunks, kUnrollD)), block(kThreads);
    auto kernel = a.param_dtype == CQ_F32 ? dequantize_flat_kernel<F, kBits, kGroup, true, kUnrollD>
                                          : dequantize_flat_kernel<F, kBits, kGroup, false, kUnrollD>;
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const uint32_t*>(a.input),
                       static_cast<u32x4*>(a.output), a.scale_in, a.param_dtype, a.num_chunks);
    return hipGetLastError();
}

template <class F, int kGroup>
hipError_t scales_launch(hipStream_t s, const FlatArgs& a) {
    dim3 grid(grid_for(a.num_chunks, kUnrollQ)), block(kThreads);
    hipLaunchKernelGGL((scales_flat_kernel<F, kGroup, kUnrollQ>), grid, block, 0, s,
                       static_cast<const u32x4*>(a.input), a.scale_out, a.num_chunks,
                       a.range.hi - a.range.lo);
    return hipGetLastError();
}

#define CQ_SWITCH_GROUP(G, ...)                          \
    switch (G) {                                         \
        case 0: { constexpr int kG = 0; __VA_ARGS__; }   \
        case 1: { constexpr int kG = 1; __VA_ARGS__; }   \
        case 2: { constexpr int kG = 2; __VA_ARGS__; }   \
        case 4: { constexpr int kG = 4; __VA_ARGS__; }   \
        case 8: { constexpr int kG = 8; __VA_ARGS__; }   \
        case 16: { constexpr int kG = 16; __VA_ARGS__; } \
        case 32: { constexpr int kG = 32; __VA_ARGS__; } \
        default: return hipErrorInvalidValue;            \
    }

#define CQ_SWITCH_BITS(B, ...)                          \
    switch (B) {                                        \
        case 2: { constexpr int kB = 2; __VA_ARGS__; }  \
        case 4: { constexpr int kB = 4; __VA_ARGS__; }  \
        case 8: { constexpr int kB = 8; __VA_ARGS__; }  \
        default: return hipErrorInvalidValue;           \
    }

#define CQ_SWITCH_DTYPE(D, ...)                              \
    switch (D) {                                             \
        case CQ_F32: { using kF = F32; __VA_ARGS__; }        \
        case CQ_BF16: { using kF = BF16; __VA_ARGS__; }      \
        case CQ_F16: { using kF = F16; __VA_ARGS__; }        \
        default: return hipErrorInvalidValue;                \
    }

}  // namespace

bool flat_block_supported(int dtype, uint32_t block) { return group_of(dtype, block) >= 0; }

hipError_t launch_quantize_flat(hipStream_t s, int dtype, int bits, ScaleSource src, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    int g = group_of(dtype, a.block);
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return quantize_launch<kF, kB, kG>(s, src, a))))
}

hipError_t launch_dequantize_flat(hipStream_t s, int dtype, int bits, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    int g = group_of(dtype, a.block);
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return dequantize_launch<kF, kB, kG>(s, a))))
}

hipError_t launch_scales_flat(hipStream_t s, int dtype, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    int g = group_of(dtype, a.block);
    if (g <= 0) return hipErrorInvalidValue;
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_GROUP(g, if constexpr (kG > 0) return scales_launch<kF, kG>(s, a); else return hipErrorInvalidValue))
}

hipError_t launch_absmax_partials(hipStream_t s, int dtype, const void* input, uint64_t num_elems,
                                  float* partials, uint32_t* num_partials) {
    uint64_t per_chunk = dtype == CQ_F32 ? 4 : 8;
    uint64_t chunks = num_elems / per_chunk;
    uint64_t want = (chunks + kThreads * 4 - 1) / (kThreads * 4);
    uint32_t grid = static_cast<uint32_t>(want < 1 ? 1 : (want > kMaxPartials ? kMaxPartials : want));
    *num_partials = grid;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((absmax_partials_kernel<kF>), dim3(grid), dim3(kThreads), 0, s,
                                              input, num_elems, partials);
                    return hipGetLastError())
}

hipError_t launch_tensor_scale(hipStream_t s, int f_dtype, int out_dtype, const float* partials,
                               uint32_t num_partials, Range range, void* out) {
    hipLaunchKernelGGL(tensor_scale_kernel, dim3(1), dim3(kThreads), 0, s, partials, num_partials,
                       range.hi - range.lo, f_dtype, out_dtype, out);
    return hipGetLastError();
}

}  // namespace cq
