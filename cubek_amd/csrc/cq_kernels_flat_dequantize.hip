// Launchers of the flat dequantize kernels of one float type and one width of codes.  The Makefile compiles this
// file nine times (-DCQ_TU_FLOAT=F32|BF16|F16, -DCQ_TU_BITS=2|4|8), each into an object of its own: the build runs
// in parallel, and a process loads the kernels of the float types and widths it uses only.
#include "cq_kernels_flat_launch.hpp"

#ifndef CQ_TU_FLOAT
#define CQ_TU_FLOAT F32
#endif
#ifndef CQ_TU_BITS
#define CQ_TU_BITS 4
#endif

namespace cq {
namespace {

template <class F, int kBits, int kGroup, int kEnc>
hipError_t dequantize_launch_enc(hipStream_t s, const FlatArgs& a) {
    auto in = static_cast<const char*>(a.input);
    auto out = static_cast<char*>(a.output);
    constexpr int kU = kUnrollD<F, kBits, kGroup>;
    [[maybe_unused]] constexpr uint64_t kInChunk = F::kPerChunk * kBits / 8;  // stored bytes per chunk
    [[maybe_unused]] const uint64_t div = kGroup == 0 ? 1 : (a.any_group != 0 ? a.any_group : kGroup);  // chunks per scale
    [[maybe_unused]] const uint64_t param_bytes = kGroup == 0 ? 0 : (a.param_dtype == CQ_F32 ? 4 : 2);
#if CQ_TU_SAME
    // this object: the whole tiles of a contiguous run, parameters typed like the tensor
    if constexpr (F::kBytes == 2 && whole_tiles_for(kGroup)) {
        hipLaunchKernelGGL((dequantize_flat_kernel<F, kBits, kGroup, kU, kThreads, kEnc, F::kDtype>), dim3(a.whole_grid),
                           dim3(kThreads), 0, s, reinterpret_cast<const uint32_t*>(in), reinterpret_cast<u32x4*>(out), a.scale_in,
                           0ull, static_cast<uint64_t>(a.whole_grid) * kThreads * kU);
        return hipGetLastError();
    } else {
        return hipErrorInvalidValue;
    }
#else
    hipError_t same = hipSuccess;
    const hipError_t e = launch_flat(
        a, F::kDtype, kU,
        [&](uint32_t grid, uint64_t) {
            if (a.param_dtype != CQ_F32) {  // a contiguous run, parameters typed like the tensor
                FlatArgs b = a;
                b.whole_grid = grid;
                same = dequantize_flat_same<F>(s, kBits, b);
            } else if (a.rows > 1) {
                if constexpr (whole_steps_for(kGroup))
                    hipLaunchKernelGGL((dequantize_flat_rows_kernel<F, kBits, kGroup, kU, kThreads, kEnc>), dim3(grid), dim3(kThreads),
                                       0, s, reinterpret_cast<const uint32_t*>(in), reinterpret_cast<u32x4*>(out), a.scale_in, 0u,
                                       flat_rows(a));
            } else {
                if constexpr (whole_tiles_for(kGroup))
                    hipLaunchKernelGGL((dequantize_flat_kernel<F, kBits, kGroup, kU, kThreads, kEnc>), dim3(grid), dim3(kThreads), 0,
                                       s, reinterpret_cast<const uint32_t*>(in), reinterpret_cast<u32x4*>(out), a.scale_in, 0ull,
                                       static_cast<uint64_t>(grid) * kThreads * kU);
            }
        },
        [&](const LaneRows& rows, uint32_t tile_begin, uint32_t grid, RunOffsets off) {
            hipLaunchKernelGGL((dequantize_flat_lanes_kernel<F, kBits, lanes_group(kGroup), kU, kThreads, kEnc>), dim3(grid), dim3(kThreads), 0,
                               s, reinterpret_cast<const uint32_t*>(in + off.chunks * kInChunk),
                               reinterpret_cast<u32x4*>(out + off.chunks * 16),
                               static_cast<const char*>(a.scale_in) + off.chunks / div * param_bytes, a.param_dtype, tile_begin,
                               with_group(rows, kGroup, a.any_group));
        });
    return e != hipSuccess ? e : same;
#endif
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

#if CQ_TU_SAME
hipError_t CQ_DEQUANTIZE_FLAT_SAME_TU(CQ_TU_FLOAT)(hipStream_t s, int bits, const FlatArgs& a) {
#else
hipError_t CQ_DEQUANTIZE_FLAT_TU(CQ_TU_FLOAT, CQ_TU_BITS)(hipStream_t s, const FlatArgs& a) {
    constexpr int bits = CQ_TU_BITS;
#endif
    int g = group_of(CQ_TU_FLOAT::kDtype, a.block);
    FlatArgs b = a;
    if (g < 0 && (b.any_group = any_group_of(CQ_TU_FLOAT::kDtype, a.block)) != 0) g = shape_group_of(b.any_group);  // lane by lane
#if CQ_TU_SAME
    CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return (dequantize_launch<CQ_TU_FLOAT, kB, kG>(s, b))))
#else
    CQ_SWITCH_GROUP(g, return (dequantize_launch<CQ_TU_FLOAT, bits, kG>(s, b)))
#endif
}

}  // namespace cq
