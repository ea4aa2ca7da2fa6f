// Launchers of the flat (contiguous) quantize kernels that read given scales.
#include "cq_kernels_flat_launch.hpp"

namespace cq {

hipError_t launch_quantize_flat_given(hipStream_t s, int dtype, int bits, const FlatArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    int g = group_of(dtype, a.block);
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_BITS(bits, CQ_SWITCH_GROUP(g, return (quantize_launch<kF, kB, kG, true>(s, ScaleSource::Given, a)))))
}

}  // namespace cq
