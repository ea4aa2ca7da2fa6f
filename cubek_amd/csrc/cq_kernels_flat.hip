// Launchers of the flat (contiguous) kernels: block scales, the per-tensor abs-max, and the dispatch of
// quantize and dequantize to the per-type launchers of cq_kernels_flat_quantize.hip and
// cq_kernels_flat_dequantize.hip.
#include "cq_kernels_flat_launch.hpp"

namespace cq {
namespace {

template <class F, int kGroup>
hipError_t scales_launch(hipStream_t s, const FlatArgs& a) {
    dim3 grid(grid_for(a.num_chunks, kUnrollQ)), block(kThreads);
    if (a.lanes.levels > 0) {
        hipLaunchKernelGGL((scales_flat_lanes_kernel<F, kGroupRt, kUnrollQ, kThreads>), dim3(lanes_grid(a, kUnrollQ)), block, 0, s,
                           static_cast<const u32x4*>(a.input), a.scale_out, quant_params(a.range), with_group(lane_rows(a), kGroup));
    } else if (a.rows > 1) {
        const FlatRows rows = flat_rows(a);
        hipLaunchKernelGGL((scales_flat_rows_kernel<F, kGroup, kUnrollQ, kThreads>), dim3((rows.total_steps + kUnrollQ - 1) / kUnrollQ),
                           block, 0, s, static_cast<const u32x4*>(a.input), a.scale_out, quant_params(a.range), rows);
    } else {
        hipLaunchKernelGGL((scales_flat_kernel<F, kGroup, kUnrollQ, kThreads>), grid, block, 0, s,
                           static_cast<const u32x4*>(a.input), a.scale_out, a.num_chunks,
                           quant_params(a.range));
    }
    return hipGetLastError();
}

}  // namespace

bool flat_block_supported(int dtype, uint32_t block) { return group_of(dtype, block) >= 0; }
bool flat_block_supported_with_scales(int dtype, uint32_t block) { return group_of(dtype, block) >= 0 || any_group_of(dtype, block) != 0; }

// mirrors launch_flat(): whole tiles of a run exist for parameters typed f32 or like the float tensor, whole steps
// of pitched rows for f32 parameters
uint32_t flat_family(const FlatArgs& a, int f_dtype) {
    const bool p32 = a.param_dtype == CQ_F32 || a.output == nullptr;  // scale production has no stored parameters
    if (a.lanes.levels > 0 || any_group_of(f_dtype, a.block) != 0 || a.lanes_only) return CQ_FAMILY_FLAT_LANES;
    const int group = group_of(f_dtype, a.block);
    if (a.rows > 1) return p32 && whole_steps_for(group) && a.num_chunks % kThreads == 0 ? CQ_FAMILY_FLAT_ROWS : CQ_FAMILY_FLAT_LANES;
    return (p32 || a.param_dtype == f_dtype) && whole_tiles_for(group) && a.num_chunks >= static_cast<uint64_t>(kThreads) * 4
               ? CQ_FAMILY_FLAT
               : CQ_FAMILY_FLAT_LANES;
}

// the objects of cq_kernels_flat_quantize.hip, by float type, family of scale sources and width of the codes
#define CQ_QUANTIZE_BY_BITS(f, g)                                              \
    switch (bits) {                                                            \
        case 2: return CQ_QUANTIZE_FLAT_TU(f, g, 2)(s, src, a);                \
        case 4: return CQ_QUANTIZE_FLAT_TU(f, g, 4)(s, src, a);                \
        case 8: return CQ_QUANTIZE_FLAT_TU(f, g, 8)(s, src, a);                \
        default: return hipErrorInvalidValue;                                  \
    }
hipError_t launch_quantize_flat(hipStream_t s, int dtype, int bits, ScaleSource src, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    const bool given = src == ScaleSource::Given || src == ScaleSource::Stored;  // the objects that read scales
    switch (dtype) {
        case CQ_F32:
            if (given) CQ_QUANTIZE_BY_BITS(F32, 1) else CQ_QUANTIZE_BY_BITS(F32, 0)
        case CQ_BF16:
            if (given) CQ_QUANTIZE_BY_BITS(BF16, 1) else CQ_QUANTIZE_BY_BITS(BF16, 0)
        case CQ_F16:
            if (given) CQ_QUANTIZE_BY_BITS(F16, 1) else CQ_QUANTIZE_BY_BITS(F16, 0)
        default: return hipErrorInvalidValue;
    }
}
#undef CQ_QUANTIZE_BY_BITS

#define CQ_DEQUANTIZE_BY_BITS(f)                                               \
    switch (bits) {                                                            \
        case 2: return CQ_DEQUANTIZE_FLAT_TU(f, 2)(s, a);                      \
        case 4: return CQ_DEQUANTIZE_FLAT_TU(f, 4)(s, a);                      \
        case 8: return CQ_DEQUANTIZE_FLAT_TU(f, 8)(s, a);                      \
        default: return hipErrorInvalidValue;                                  \
    }
hipError_t launch_dequantize_flat(hipStream_t s, int dtype, int bits, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    switch (dtype) {
        case CQ_F32: CQ_DEQUANTIZE_BY_BITS(F32)
        case CQ_BF16: CQ_DEQUANTIZE_BY_BITS(BF16)
        case CQ_F16: CQ_DEQUANTIZE_BY_BITS(F16)
        default: return hipErrorInvalidValue;
    }
}
#undef CQ_DEQUANTIZE_BY_BITS

hipError_t launch_scales_flat(hipStream_t s, int dtype, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    int g = group_of(dtype, a.block);
    if (g <= 0) return hipErrorInvalidValue;
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_GROUP(g, if constexpr (kG > 0) return scales_launch<kF, kG>(s, a); else return hipErrorInvalidValue))
}

hipError_t launch_absmax_partials(hipStream_t s, int dtype, const void* input, uint64_t num_elems,
                                  float* partials, uint32_t* num_partials) {
    // At most kMaxPartials workgroups (pass 2 re-reads every partial in every
    // workgroup), so they are fat: 1024 lanes x 4 loads = 64 KiB in flight each.
    constexpr int kReduceThreads = 1024, kReduceUnroll = 4;
    const uint64_t per_chunk = dtype == CQ_F32 ? 4 : 8;
    const uint64_t chunks = num_elems / per_chunk;
    const uint64_t per_group = static_cast<uint64_t>(kReduceThreads) * kReduceUnroll;
    const uint64_t want = (chunks + per_group - 1) / per_group;
    uint32_t grid = static_cast<uint32_t>(want < 1 ? 1 : (want > kMaxPartials ? kMaxPartials : want));
    if (grid > 8) grid = (grid + 7) & ~7u;  // a multiple of the 8 XCDs: block b of the tensor is read on XCD b % 8
    const bool is_aligned = (reinterpret_cast<uintptr_t>(input) & 15u) == 0;
    *num_partials = grid;
    CQ_SWITCH_DTYPE(dtype,
                    auto kernel = is_aligned ? absmax_partials_kernel<kF, kReduceThreads, kReduceUnroll, true>
                                             : absmax_partials_kernel<kF, kReduceThreads, kReduceUnroll, false>;
                    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kReduceThreads), 0, s, input, num_elems, partials);
                    return hipGetLastError())
}

hipError_t launch_tensor_scale(hipStream_t s, int f_dtype, int out_dtype, const float* partials,
                               uint32_t num_partials, Range range, void* out) {
    hipLaunchKernelGGL(tensor_scale_kernel<kThreads>, dim3(1), dim3(kThreads), 0, s, partials, num_partials,
                       range.hi - range.lo, f_dtype, out_dtype, out);
    return hipGetLastError();
}

}  // namespace cq
