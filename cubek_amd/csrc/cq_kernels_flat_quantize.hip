// Launchers of the flat quantize kernels of one float type, one family of scale sources and one width of codes.  The
// Makefile compiles this file eighteen times (-DCQ_TU_FLOAT=F32|BF16|F16, -DCQ_TU_GIVEN=0|1: scales produced
// in the launch, or given, -DCQ_TU_BITS=2|4|8), each into an object of its own, so that the build runs in parallel
// (in one translation unit the instantiations take minutes) and a process's first launch loads a third of a
// megabyte of code, not all of it.  Four more objects (-DCQ_TU_SAME=1, BF16 and F16, every width) hold the
// whole-tile kernels for parameters typed like the tensor.
#include "cq_kernels_flat_launch.hpp"

#ifndef CQ_TU_FLOAT
#define CQ_TU_FLOAT F32
#endif
#ifndef CQ_TU_GIVEN
#define CQ_TU_GIVEN 0
#endif
#ifndef CQ_TU_BITS
#define CQ_TU_BITS 4
#endif

namespace cq {

#if CQ_TU_SAME
hipError_t CQ_QUANTIZE_FLAT_SAME_TU(CQ_TU_FLOAT, CQ_TU_GIVEN)(hipStream_t s, int bits, ScaleSource src, const FlatArgs& a) {
#else
hipError_t CQ_QUANTIZE_FLAT_TU(CQ_TU_FLOAT, CQ_TU_GIVEN, CQ_TU_BITS)(hipStream_t s, ScaleSource src, const FlatArgs& a) {
    constexpr int bits = CQ_TU_BITS;
#endif
    int g = group_of(CQ_TU_FLOAT::kDtype, a.block);
    FlatArgs b = a;
    b.lanes_only = fields_wrap(a);
    // blocks of another whole number of chunks: lane by lane, for the launches that read their scales
    if (g < 0 && (src == ScaleSource::Given || src == ScaleSource::Stored) && (b.any_group = any_group_of(CQ_TU_FLOAT::kDtype, a.block)) != 0)
        g = shape_group_of(b.any_group);
#if CQ_TU_SAME
    CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return (quantize_launch<CQ_TU_FLOAT, kB, kG, CQ_TU_GIVEN != 0>(s, src, b))))
#else
    CQ_SWITCH_GROUP(g, return (quantize_launch<CQ_TU_FLOAT, bits, kG, CQ_TU_GIVEN != 0>(s, src, b)))
#endif
}

}  // namespace cq
