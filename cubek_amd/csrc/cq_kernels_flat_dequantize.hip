// Launchers of the flat dequantize kernels of one float type.  The Makefile compiles this file three
// times (-DCQ_TU_FLOAT=F32|BF16|F16), each into an object of its own: the build runs in parallel, and a
// process loads the kernels of the float types it uses only.
#include "cq_kernels_flat_launch.hpp"

#ifndef CQ_TU_FLOAT
#define CQ_TU_FLOAT F32
#endif

namespace cq {
namespace {

template <class F, int kBits, int kGroup, int kEnc>
hipError_t dequantize_launch_enc(hipStream_t s, const FlatArgs& a) {
    auto in = static_cast<const uint32_t*>(a.input);
    auto out = static_cast<u32x4*>(a.output);
    const bool p32 = a.param_dtype == CQ_F32;
    constexpr int kU = kUnrollD<F, kBits, kGroup>;
    if (a.lanes.levels > 0) {
        hipLaunchKernelGGL((dequantize_flat_lanes_kernel<F, kBits, kGroup, kU, kThreads, kEnc>), dim3(lanes_grid(a, kU)),
                           dim3(kThreads), 0, s, in, out, a.scale_in, a.param_dtype, lane_rows(a));
        return hipGetLastError();
    }
    if (a.rows > 1)
        return launch_row_steps(a, kU, [&](bool checked, uint32_t grid, uint32_t step_begin) {
            auto kernel = checked ? (p32 ? dequantize_flat_rows_kernel<F, kBits, kGroup, true, kU, kThreads, true, kEnc>
                                         : dequantize_flat_rows_kernel<F, kBits, kGroup, false, kU, kThreads, true, kEnc>)
                                  : (p32 ? dequantize_flat_rows_kernel<F, kBits, kGroup, true, kU, kThreads, false, kEnc>
                                         : dequantize_flat_rows_kernel<F, kBits, kGroup, false, kU, kThreads, false, kEnc>);
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, s, in, out, a.scale_in, a.param_dtype, step_begin,
                               flat_rows(a));
        });
    return launch_tiles(a.num_chunks, kU, [&](bool checked, uint32_t grid, uint64_t begin, uint64_t end) {
        auto kernel = checked ? (p32 ? dequantize_flat_kernel<F, kBits, kGroup, true, kU, kThreads, true, kEnc>
                                     : dequantize_flat_kernel<F, kBits, kGroup, false, kU, kThreads, true, kEnc>)
                              : (p32 ? dequantize_flat_kernel<F, kBits, kGroup, true, kU, kThreads, false, kEnc>
                                     : dequantize_flat_kernel<F, kBits, kGroup, false, kU, kThreads, false, kEnc>);
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, s, in, out, a.scale_in, a.param_dtype, begin, end);
    });
}

template <class F, int kBits, int kGroup>
hipError_t dequantize_launch(hipStream_t s, const FlatArgs& a) {
    switch (a.encoding) {
        case kEncInt: return dequantize_launch_enc<F, kBits, kGroup, kEncInt>(s, a);
        case kEncE4M3:
            if constexpr (kBits == 8) return dequantize_launch_enc<F, 8, kGroup, kEncE4M3>(s, a);
            break;
        case kEncE5M2:
            if constexpr (kBits == 8) return dequantize_launch_enc<F, 8, kGroup, kEncE5M2>(s, a);
            break;
        case kEncE2M1:
            if constexpr (kBits == 4) return dequantize_launch_enc<F, 4, kGroup, kEncE2M1>(s, a);
            break;
    }
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t CQ_DEQUANTIZE_FLAT_TU(CQ_TU_FLOAT)(hipStream_t s, int bits, const FlatArgs& a) {
    int g = group_of(CQ_TU_FLOAT::kDtype, a.block);
    CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return (dequantize_launch<CQ_TU_FLOAT, kB, kG>(s, a))))
}

}  // namespace cq
