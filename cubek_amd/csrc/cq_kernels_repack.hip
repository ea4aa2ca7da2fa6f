// Strided quantized tensor -> contiguous tensor packed along the last dimension:
// the re-packing cubek-matmul asks of cubecl-std's into_contiguous_packed before it
// hands quantized operands to its kernels (crates/cubek-matmul/src/base.rs:505-529).
// Stored element `pos` of the output gathers the logical values pos*P .. pos*P+P-1
// (P values per stored element, value 0 in the low bits); the input holds P values
// per element along `packed_dim` and is addressed through its strides.
#include "cq_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;

// One thread per output element, any rank and strides.
template <class W>
__global__ __launch_bounds__(kThreads) void repack_generic_kernel(RepackArgs a) {
    const uint64_t pos = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (pos >= a.num_out) return;
    const int last = static_cast<int>(a.rank) - 1;
    const W* in = static_cast<const W*>(a.input);
    // offset of the input element that holds the first of the P logical values
    uint64_t rem = pos, base = 0;
    uint32_t sub = 0;
    for (int d = last; d >= 0; d--) {
        const uint32_t n = d == last ? a.shape[d] / a.packing : a.shape[d];
        uint64_t c = rem % n;
        rem /= n;
        if (static_cast<uint32_t>(d) == a.packed_dim) {
            if (d != last) {
                sub = static_cast<uint32_t>(c % a.packing);
                c /= a.packing;
            }
        } else if (d == last) {
            c *= a.packing;
        }
        base += c * a.strides[d];
    }
    uint32_t out;
    if (static_cast<int>(a.packed_dim) == last) {
        out = in[base];  // same packing on both sides: a strided copy
    } else {
        const uint32_t mask = a.bits == 32 ? 0xffffffffu : (1u << a.bits) - 1u;
        out = 0;
        for (uint32_t k = 0; k < a.packing; k++)
            out |= ((static_cast<uint32_t>(in[base + k * a.strides[last]]) >> (sub * a.bits)) & mask) << (k * a.bits);
    }
    static_cast<W*>(a.output)[pos] = static_cast<W>(out);
}

}  // namespace

hipError_t launch_repack(hipStream_t s, const RepackArgs& a) {
    if (a.num_out == 0) return hipSuccess;
    const dim3 grid(static_cast<uint32_t>((a.num_out + kThreads - 1) / kThreads));
    if (a.elem_bytes == 4)
        hipLaunchKernelGGL((repack_generic_kernel<uint32_t>), grid, dim3(kThreads), 0, s, a);
    else
        hipLaunchKernelGGL((repack_generic_kernel<uint8_t>), grid, dim3(kThreads), 0, s, a);
    return hipGetLastError();
}

}  // namespace cq
