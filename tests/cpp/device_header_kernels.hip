// Consumer kernels built on include/cubek_quant_device.hpp only, behind a small C interface that the
// pytest suite drives (tests/test_gpu_device_header.py): every function of the header runs on the
// committed fixtures and is compared with their expected values, not with the library.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cubek_quant_device.hpp"

namespace dev = cubek_quant::device;

namespace {

// kF value (exactly representable) -> storage bits
template <dev::Float kF>
__device__ __forceinline__ void store_value(void* out, uint64_t i, float v) {
    if constexpr (kF == dev::Float::F32)
        static_cast<float*>(out)[i] = v;
    else if constexpr (kF == dev::Float::F16)
        static_cast<_Float16*>(out)[i] = static_cast<_Float16>(v);
    else
        static_cast<__bf16*>(out)[i] = static_cast<__bf16>(v);
}

// dequantize-on-read of a whole packed tensor, one word per thread
template <dev::Float kF, int kBits, class FS, bool kPairs>
__global__ void dequantize_packed_kernel(const uint32_t* words, const FS* scales, dev::ScalesLayout layout,
                                         uint64_t num_words, void* out) {
    constexpr int nq = 32 / kBits;
    const uint64_t p = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= num_words) return;
    if constexpr (kPairs && kF != dev::Float::F32) {
        uint32_t pairs[nq / 2];
        dev::dequantize_symmetric_packed_value_pairs<kF, kBits>(words[p], scales[layout.to_source_pos(p * nq)], pairs);
        for (int i = 0; i < nq / 2; i++) static_cast<uint32_t*>(out)[p * (nq / 2) + i] = pairs[i];
    } else {
        float v[nq];
        dev::dequantize_symmetric_packed_values<kF, kBits>(p, words, scales, layout, v);
        for (int i = 0; i < nq; i++) store_value<kF>(out, p * nq + i, v[i]);
    }
}

// the same for the native store, 32 bits per thread
template <dev::Float kF, dev::Native kNative, class FS>
__global__ void dequantize_native_kernel(const uint32_t* words, const FS* scales, dev::ScalesLayout layout,
                                         uint64_t num_words, void* out) {
    constexpr int kN = dev::native_values_per_word<kNative>();
    const uint64_t p = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= num_words) return;
    float v[kN];
    dev::dequantize_symmetric_native_values<kF, kNative>(p, words, scales, layout, v);
    for (int i = 0; i < kN; i++) store_value<kF>(out, p * kN + i, v[i]);
}

// ... and through dequantize_symmetric_native_value_pairs (16-bit float types; e4m3, e5m2, e2m1x2)
template <dev::Float kF, dev::Native kNative, class FS>
__global__ void dequantize_native_pairs_kernel(const uint32_t* words, const FS* scales, dev::ScalesLayout layout,
                                               uint64_t num_words, void* out) {
    constexpr int kN = dev::native_values_per_word<kNative>();
    const uint64_t p = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= num_words) return;
    uint32_t pairs[kN / 2];
    dev::dequantize_symmetric_native_value_pairs<kF, kNative>(words[p], scales[layout.to_source_pos(p * kN)], pairs);
    for (int i = 0; i < kN / 2; i++) static_cast<uint32_t*>(out)[p * (kN / 2) + i] = pairs[i];
}

// scale index of every element of a [batches, rows, cols] tensor through GlobalScaleLayout
template <uint32_t kBR, uint32_t kBC>
__global__ void scale_pos_kernel(dev::GlobalScaleLayout<kBR, kBC> layout, uint32_t batches, uint32_t rows, uint32_t cols,
                                 uint32_t* out) {
    const uint32_t col = blockIdx.x * blockDim.x + threadIdx.x, row = blockIdx.y, batch = blockIdx.z;
    if (col < cols) out[(static_cast<uint64_t>(batch) * rows + row) * cols + col] = layout.to_source_pos(batch, row, col);
}

// element index -> scale index and block-start flag through ScalesLayout, on the device
__global__ void scales_layout_kernel(dev::ScalesLayout layout, uint64_t n, uint64_t* pos, uint8_t* start) {
    const uint64_t e = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= n) return;
    pos[e] = layout.to_source_pos(e);
    start[e] = layout.is_block_start(e);
}

dim3 grid_for(uint64_t n) { return dim3(static_cast<uint32_t>((n + 255) / 256)); }

template <dev::Float kF, int kBits, class FS>
void launch_packed(bool pairs, const uint32_t* words, const void* scales, const dev::ScalesLayout& l, uint64_t n, void* out) {
    if (pairs)
        hipLaunchKernelGGL((dequantize_packed_kernel<kF, kBits, FS, true>), grid_for(n), dim3(256), 0, 0, words,
                           static_cast<const FS*>(scales), l, n, out);
    else
        hipLaunchKernelGGL((dequantize_packed_kernel<kF, kBits, FS, false>), grid_for(n), dim3(256), 0, 0, words,
                           static_cast<const FS*>(scales), l, n, out);
}
template <dev::Float kF, int kBits>
int packed_param(int param, bool pairs, const uint32_t* words, const void* scales, const dev::ScalesLayout& l, uint64_t n,
                 void* out) {
    switch (param) {
        case 0: launch_packed<kF, kBits, float>(pairs, words, scales, l, n, out); return 0;
        case 1: launch_packed<kF, kBits, _Float16>(pairs, words, scales, l, n, out); return 0;
        case 2: launch_packed<kF, kBits, __bf16>(pairs, words, scales, l, n, out); return 0;
    }
    return -1;
}
template <dev::Float kF>
int packed_bits(int bits, int param, bool pairs, const uint32_t* words, const void* scales, const dev::ScalesLayout& l,
                uint64_t n, void* out) {
    switch (bits) {
        case 2: return packed_param<kF, 2>(param, pairs, words, scales, l, n, out);
        case 4: return packed_param<kF, 4>(param, pairs, words, scales, l, n, out);
        case 8: return packed_param<kF, 8>(param, pairs, words, scales, l, n, out);
    }
    return -1;
}

template <dev::Float kF, dev::Native kNative>
int native_param(int param, const uint32_t* words, const void* scales, const dev::ScalesLayout& l, uint64_t n, void* out) {
    switch (param) {
        case 0:
            hipLaunchKernelGGL((dequantize_native_kernel<kF, kNative, float>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const float*>(scales), l, n, out);
            return 0;
        case 1:
            hipLaunchKernelGGL((dequantize_native_kernel<kF, kNative, _Float16>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const _Float16*>(scales), l, n, out);
            return 0;
        case 2:
            hipLaunchKernelGGL((dequantize_native_kernel<kF, kNative, __bf16>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const __bf16*>(scales), l, n, out);
            return 0;
    }
    return -1;
}
template <dev::Float kF>
int native_store(int native, int param, const uint32_t* words, const void* scales, const dev::ScalesLayout& l, uint64_t n,
                 void* out) {
    switch (native) {
        case 0: return native_param<kF, dev::Native::I8>(param, words, scales, l, n, out);
        case 1: return native_param<kF, dev::Native::E4M3>(param, words, scales, l, n, out);
        case 2: return native_param<kF, dev::Native::E5M2>(param, words, scales, l, n, out);
        case 3: return native_param<kF, dev::Native::E2M1x2>(param, words, scales, l, n, out);
    }
    return -1;
}

template <dev::Float kF, dev::Native kNative>
int native_pairs_param(int param, const uint32_t* words, const void* scales, const dev::ScalesLayout& l, uint64_t n, void* out) {
    switch (param) {
        case 0:
            hipLaunchKernelGGL((dequantize_native_pairs_kernel<kF, kNative, float>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const float*>(scales), l, n, out);
            return 0;
        case 1:
            hipLaunchKernelGGL((dequantize_native_pairs_kernel<kF, kNative, _Float16>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const _Float16*>(scales), l, n, out);
            return 0;
        case 2:
            hipLaunchKernelGGL((dequantize_native_pairs_kernel<kF, kNative, __bf16>), grid_for(n), dim3(256), 0, 0, words,
                               static_cast<const __bf16*>(scales), l, n, out);
            return 0;
    }
    return -1;
}
template <dev::Float kF>
int native_pairs_store(int native, int param, const uint32_t* words, const void* scales, const dev::ScalesLayout& l,
                       uint64_t n, void* out) {
    switch (native) {
        case 1: return native_pairs_param<kF, dev::Native::E4M3>(param, words, scales, l, n, out);
        case 2: return native_pairs_param<kF, dev::Native::E5M2>(param, words, scales, l, n, out);
        case 3: return native_pairs_param<kF, dev::Native::E2M1x2>(param, words, scales, l, n, out);
    }
    return -1;
}

int finish() { return hipGetLastError() == hipSuccess && hipDeviceSynchronize() == hipSuccess ? 0 : -2; }

}  // namespace

extern "C" {

// float_type / param: 0 f32, 1 f16, 2 bf16 (cq_dtype).  values_shape is the QUANTIZED tensor's shape.
// `pairs` != 0: through dequantize_symmetric_packed_value_pairs (16-bit float types).
int dh_dequantize_packed(int float_type, int bits, int param, int pairs, const uint32_t* words, const void* scales,
                         const uint64_t* values_shape, uint32_t rank, const uint64_t* scales_strides,
                         const uint8_t* block, uint32_t block_rank, uint64_t num_words, void* out) {
    const dev::ScalesLayout l = dev::scales_layout(values_shape, rank, 32u / bits, scales_strides, block, block_rank);
    int rc = -1;
    switch (float_type) {
        case 0: rc = packed_bits<dev::Float::F32>(bits, param, pairs != 0, words, scales, l, num_words, out); break;
        case 1: rc = packed_bits<dev::Float::F16>(bits, param, pairs != 0, words, scales, l, num_words, out); break;
        case 2: rc = packed_bits<dev::Float::BF16>(bits, param, pairs != 0, words, scales, l, num_words, out); break;
    }
    return rc ? rc : finish();
}

// native: 0 i8, 1 e4m3, 2 e5m2, 3 e2m1x2; `num_words` counts 32-bit units of the stored tensor.
int dh_dequantize_native(int float_type, int native, int param, const uint32_t* words, const void* scales,
                         const uint64_t* values_shape, uint32_t rank, const uint64_t* scales_strides,
                         const uint8_t* block, uint32_t block_rank, uint64_t num_words, void* out) {
    const dev::ScalesLayout l =
        dev::scales_layout(values_shape, rank, native == 3 ? 2u : 1u, scales_strides, block, block_rank);
    int rc = -1;
    switch (float_type) {
        case 0: rc = native_store<dev::Float::F32>(native, param, words, scales, l, num_words, out); break;
        case 1: rc = native_store<dev::Float::F16>(native, param, words, scales, l, num_words, out); break;
        case 2: rc = native_store<dev::Float::BF16>(native, param, words, scales, l, num_words, out); break;
    }
    return rc ? rc : finish();
}

// The same through dequantize_symmetric_native_value_pairs: float_type 1 or 2, native 1, 2 or 3.
int dh_dequantize_native_pairs(int float_type, int native, int param, const uint32_t* words, const void* scales,
                               const uint64_t* values_shape, uint32_t rank, const uint64_t* scales_strides,
                               const uint8_t* block, uint32_t block_rank, uint64_t num_words, void* out) {
    const dev::ScalesLayout l =
        dev::scales_layout(values_shape, rank, native == 3 ? 2u : 1u, scales_strides, block, block_rank);
    int rc = -1;
    switch (float_type) {
        case 1: rc = native_pairs_store<dev::Float::F16>(native, param, words, scales, l, num_words, out); break;
        case 2: rc = native_pairs_store<dev::Float::BF16>(native, param, words, scales, l, num_words, out); break;
    }
    return rc ? rc : finish();
}

// GlobalScaleLayout over [batches, rows, cols] for a few compile-time block shapes; out[b][r][c] = scale index.
int dh_global_scale_pos(uint32_t block_rows, uint32_t block_cols, uint32_t stride_batch, uint32_t stride_row,
                        uint32_t stride_col, uint32_t batches, uint32_t rows, uint32_t cols, uint32_t* out) {
    const dim3 grid((cols + 63) / 64, rows, batches), block(64);
#define DH_CASE(BR, BC)                                                                                          \
    if (block_rows == BR && block_cols == BC) {                                                                  \
        dev::GlobalScaleLayout<BR, BC> l;                                                                        \
        l.stride_batch = stride_batch, l.stride_row = stride_row, l.stride_col = stride_col;                     \
        hipLaunchKernelGGL((scale_pos_kernel<BR, BC>), grid, block, 0, 0, l, batches, rows, cols, out);          \
        return finish();                                                                                         \
    }
    DH_CASE(0, 0) DH_CASE(1, 32) DH_CASE(1, 24) DH_CASE(128, 128) DH_CASE(3, 16) DH_CASE(16, 1)
#undef DH_CASE
    return -1;
}

// ScalesLayout on the device: pos[e], start[e] for e < n (shape = the quantized tensor's, as above).
int dh_scales_layout(const uint64_t* values_shape, uint32_t rank, uint32_t num_quants, const uint64_t* scales_strides,
                     const uint8_t* block, uint32_t block_rank, uint64_t n, uint64_t* pos, uint8_t* start) {
    const dev::ScalesLayout l = dev::scales_layout(values_shape, rank, num_quants, scales_strides, block, block_rank);
    hipLaunchKernelGGL(scales_layout_kernel, grid_for(n), dim3(256), 0, 0, l, n, pos, start);
    return finish();
}

// The same functions on the host (they are __host__ __device__): no GPU needed.
uint64_t dh_host_scale_pos(const uint64_t* values_shape, uint32_t rank, uint32_t num_quants, const uint64_t* scales_strides,
                           const uint8_t* block, uint32_t block_rank, uint64_t pos) {
    return dev::scales_layout(values_shape, rank, num_quants, scales_strides, block, block_rank).to_source_pos(pos);
}
int dh_host_is_block_start(const uint64_t* values_shape, uint32_t rank, uint32_t num_quants, const uint64_t* scales_strides,
                           const uint8_t* block, uint32_t block_rank, uint64_t pos) {
    return dev::scales_layout(values_shape, rank, num_quants, scales_strides, block, block_rank).is_block_start(pos);
}
uint32_t dh_host_fast_div(uint32_t n, uint32_t d) { return dev::FastDivmod(d).div(n); }

}  // extern "C"
