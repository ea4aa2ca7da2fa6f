// y = dequantize(W) * x for a quantized weight matrix that is read once, in its packed form: the
// consumer side of the packed format ("weight-load path").  It stands where the reference's matmul
// takes a quantized operand (MatmulInputHandle::Quantized, crates/cubek-matmul/src/base.rs:309-317)
// and dequantizes it while loading, with the crate's public device functions
// (crates/cubek-quant/src/dequantize.rs:20-79) and a 2-D scale lookup
// (crates/cubek-matmul/src/components/global/memory/layout.rs:371-455).
//
// Everything that touches the packed format below comes from the public device header
// (include/cubek_quant_device.hpp): the kernels are what a user of that header would write.
// A weight enters the products as the value cq_dequantize would store, F(F(scale) * F(code)),
// rounded to the float type F of x; products are accumulated in f32.
//
// HBM bytes per weight: bits / 8 for the code plus one scale per block (2.625 bits -> 0.625 B per
// weight for 4-bit codes with f32 scales on blocks of 32); x and y are negligible.  The roofline is HBM.
#include <hip/hip_runtime.h>

#include "../../include/cubek_quant_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

namespace dev = cubek_quant::device;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <dev::Float kF>
struct Elem;
template <>
struct Elem<dev::Float::F32> { using T = float; };
template <>
struct Elem<dev::Float::F16> { using T = _Float16; };
template <>
struct Elem<dev::Float::BF16> { using T = __bf16; };

// a[0] * b[0] + a[1] * b[1] + acc over packed pairs of a 16-bit float type, in f32
template <dev::Float kF>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (kF == dev::Float::BF16) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
    } else {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// v + (v of the lane the DPP control selects); lanes outside the masks or without a source add 0
template <int kCtrl, int kRowMask = 0xf>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, 0xf, true));
}
// Sum over the 64 lanes of a wave, valid in lane 63 only: an inclusive scan inside each row of 16 lanes
// (row_shr 1, 2, 4, 8), then the row totals handed on (row_bcast:15 into rows 1 and 3, row_bcast:31 into
// rows 2 and 3).  Six VALU instructions, no LDS.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v = dpp_add<0x111>(v);
    v = dpp_add<0x112>(v);
    v = dpp_add<0x114>(v);
    v = dpp_add<0x118>(v);
    v = dpp_add<0x142, 0xa>(v);
    v = dpp_add<0x143, 0xc>(v);
    return v;
}

__device__ __forceinline__ void store_y(int dtype, void* y, uint64_t i, float v) {
    if (dtype == CQ_F32)
        static_cast<float*>(y)[i] = v;
    else if (dtype == CQ_F16)
        static_cast<_Float16*>(y)[i] = static_cast<_Float16>(v);
    else
        static_cast<__bf16*>(y)[i] = static_cast<__bf16>(v);
}

// ---- streaming kernel: 16-bit float types, 1-D blocks of 32 values, 4-bit codes ---------------------
// A lane owns one block per row: four words (one 16-byte load) and one scale.  A wave covers a strip of
// 64 blocks = 2048 columns; the waves of a workgroup are the strips of a row, so the 32 values of x a lane
// needs never change: they stay in 16 registers as packed pairs while the workgroup walks its rows in
// passes of up to kRows * kChunks rows.  Inside a pass the loads of chunk c + 1 (kRows rows) are issued
// before chunk c is worked on, so memory and arithmetic overlap inside every wave; the per-lane sums of
// a pass stay in registers and meet once, at its end: six DPP additions per row, then one LDS exchange
// across the strips.  Per value: one byte-to-float conversion and one FMA
// (dequantize_symmetric_packed_value_pairs), half a v_cvt_pk, half a v_dot2.
// kRows rows of one lane: the four words of its block and the block's scale, per row
template <class FS, int kRows>
struct RowChunk {
    u32x4 w[kRows];
    FS s[kRows];
};

template <dev::Float kF, class FS, int kRows, int kChunks, int kMaxStrips>
__global__ __launch_bounds__(64 * kMaxStrips) void gemv_w4_b32_kernel(
    const uint32_t* __restrict__ words, const FS* __restrict__ scales, const void* __restrict__ x, void* __restrict__ y,
    int y_dtype, uint32_t rows, uint32_t blocks_per_row, uint32_t rows_per_group, uint64_t word_pitch,
    dev::GlobalScaleLayout<1, 32> scale_at) {
    static_assert(kChunks == 4, "the pass below is written out for four chunks");
    constexpr int kPass = kRows * kChunks;
    using Chunk = RowChunk<FS, kRows>;
    const uint32_t lane = threadIdx.x & 63u, strip = threadIdx.x >> 6, strips = blockDim.x >> 6;
    const uint32_t block = strip * 64u + lane;
    const bool live = block < blocks_per_row;
    const uint32_t b = live ? block : blocks_per_row - 1;  // idle lanes re-read the row's last block
    // this lane's 32 values of x, as 16 pairs; nothing waits for them before the first rows are on their way
    uint32_t xp[16];
    {
        const u32x4* xv = static_cast<const u32x4*>(x) + static_cast<uint64_t>(b) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u32x4 v = xv[j];
            xp[4 * j] = v[0], xp[4 * j + 1] = v[1], xp[4 * j + 2] = v[2], xp[4 * j + 3] = v[3];
        }
    }
    __shared__ float partial[kMaxStrips][kPass];
    const uint32_t row_begin = blockIdx.x * rows_per_group;
    const uint32_t row_end = min(row_begin + rows_per_group, rows);
    const u32x4* const wbase = reinterpret_cast<const u32x4*>(words) + b;
    const uint64_t wstep = word_pitch / 4;  // row pitch in 16-byte units

    // rows [first, first + kRows) of the pass; rows past the workgroup's end re-read its last row
    const auto load = [&](Chunk& c, uint32_t first) {
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            const uint32_t r = min(first + k, row_end - 1);
            c.w[k] = __builtin_nontemporal_load(wbase + r * wstep);
            c.s[k] = __builtin_nontemporal_load(scales + scale_at.to_source_pos(0, r, b * 32u));
        }
        __builtin_amdgcn_sched_barrier(0);  // loads stay where they are written: one chunk ahead of the arithmetic
    };
    // One row's share of this lane, the plain way: words, scale and x read again from memory in rolled loops
    // (few registers, little code).  Only lanes whose scale is not tame come here.
    const auto plain_row = [&](uint32_t r) {
        const uint32_t* wr = words + r * word_pitch + b * 4u;
        const FS scale = scales[scale_at.to_source_pos(0, r, b * 32u)];
        const typename Elem<kF>::T* xr = static_cast<const typename Elem<kF>::T*>(x) + b * 32u;
        float a = 0.0f;
#pragma unroll 1
        for (int j = 0; j < 4; j++) {
            float v[8];
            dev::dequantize_symmetric_packed_value<kF, 4>(wr[j], scale, v);
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const uint32_t xpair = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, xr[8 * j + i])) |
                                       static_cast<uint32_t>(__builtin_bit_cast(uint16_t, xr[8 * j + i + 1])) << 16;
                a = dot2<kF>(dev::pack_pair<kF>(v[i], v[i + 1]), xpair, a);
            }
        }
        return live ? a : 0.0f;
    };
    // rows [first, first + kRows) out of a chunk's registers into acc[0..kRows); rows past the workgroup's end
    // are skipped (the row numbers are wave-uniform, so these are scalar branches)
    const auto work = [&](const Chunk& c, uint32_t first, float* acc) {
        bool tame = true;
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            if (k > 0 && first + k >= row_end) break;
            float a = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint32_t pairs[4];
                dev::dequantize_symmetric_packed_value_pairs_tame<kF, 4>(c.w[k][j], c.s[k], pairs);
#pragma unroll
                for (int i = 0; i < 4; i++) a = dot2<kF>(pairs[i], xp[4 * j + i], a);
            }
            acc[k] = live ? a : 0.0f;  // idle lanes worked on a copy of the row's last block
            tame = tame && dev::pairs_scale_is_tame<kF>(c.s[k]);
        }
        // ordinary scales are all tame: one wave-uniform test per chunk, then straight on
        if (__builtin_amdgcn_ballot_w64(!tame) != 0) {
#pragma unroll
            for (int k = 0; k < kRows; k++)
                if (first + k < row_end && !dev::pairs_scale_is_tame<kF>(c.s[k])) acc[k] = plain_row(first + k);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // Chunks alternate between two register sets; each is re-filled, two chunks ahead, as soon as its rows have
    // been worked on, also across the end of a pass, so the stream of loads never pauses for a reduction.
    Chunk ca, cb;
    load(ca, row_begin);
    if (row_begin + kRows < row_end) load(cb, row_begin + kRows);
    for (uint32_t p0 = row_begin; p0 < row_end; p0 += kPass) {
        // which chunks exist is wave-uniform: scalar branches
        float acc[kPass];
#pragma unroll
        for (int k = 0; k < kPass; k++) acc[k] = 0.0f;
        work(ca, p0, acc);
        if (p0 + 2 * kRows < row_end) load(ca, p0 + 2 * kRows);
        if (p0 + kRows < row_end) work(cb, p0 + kRows, acc + kRows);
        if (p0 + 3 * kRows < row_end) load(cb, p0 + 3 * kRows);
        if (p0 + 2 * kRows < row_end) work(ca, p0 + 2 * kRows, acc + 2 * kRows);
        if (p0 + 4 * kRows < row_end) load(ca, p0 + 4 * kRows);  // the next pass's first chunk
        if (p0 + 3 * kRows < row_end) work(cb, p0 + 3 * kRows, acc + 3 * kRows);
        if (p0 + 5 * kRows < row_end) load(cb, p0 + 5 * kRows);
        // the pass's row sums: lane 63 of every wave holds its strip's share
#pragma unroll
        for (int k = 0; k < kPass; k++)
            if (p0 + k < row_end) acc[k] = wave_sum_to_lane63(acc[k]);
        if (lane == 63) {
#pragma unroll
            for (int k = 0; k < kPass; k++) partial[strip][k] = acc[k];
        }
        __syncthreads();
        if (threadIdx.x < kPass && p0 + threadIdx.x < row_end) {
            float v = 0.0f;
            for (uint32_t t = 0; t < strips; t++) v += partial[t][threadIdx.x];
            store_y(y_dtype, y, p0 + threadIdx.x, v);
        }
        __syncthreads();
    }
}

// ---- general kernel: every packed scheme, any block shape, any float type ------------------------
// One wave per row; lane l takes words l, l + 64, ... of the row and looks each word's scale up through the
// N-D ScalesLayout.
template <dev::Float kF, int kBits, class FS>
__global__ __launch_bounds__(256) void gemv_packed_kernel(const uint32_t* __restrict__ words, const FS* __restrict__ scales,
                                                         dev::ScalesLayout layout, const void* __restrict__ x,
                                                         void* __restrict__ y, int y_dtype, uint32_t rows,
                                                         uint32_t words_per_row, uint64_t word_pitch) {
    constexpr uint32_t nq = 32 / kBits;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const typename Elem<kF>::T* xv = static_cast<const typename Elem<kF>::T*>(x);
    float acc = 0.0f;
    for (uint32_t w = lane; w < words_per_row; w += 64) {
        float v[nq];
        const uint64_t elem = (static_cast<uint64_t>(row) * words_per_row + w) * nq;
        dev::dequantize_symmetric_packed_value<kF, kBits>(words[row * word_pitch + w], scales[layout.to_source_pos(elem)], v);
#pragma unroll
        for (uint32_t i = 0; i < nq; i++) acc = __builtin_fmaf(v[i], static_cast<float>(xv[w * nq + i]), acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) store_y(y_dtype, y, row, acc);
}

template <dev::Float kF, int kBits>
hipError_t launch_general(hipStream_t s, const GemvArgs& a, const dev::ScalesLayout& layout) {
    const dim3 grid((a.rows + 3) / 4), block(256);
    switch (a.param_dtype) {
        case CQ_F32:
            hipLaunchKernelGGL((gemv_packed_kernel<kF, kBits, float>), grid, block, 0, s, static_cast<const uint32_t*>(a.words),
                               static_cast<const float*>(a.scales), layout, a.x, a.y, a.y_dtype, a.rows, a.cols / (32 / kBits),
                               a.word_pitch);
            break;
        case CQ_F16:
            hipLaunchKernelGGL((gemv_packed_kernel<kF, kBits, _Float16>), grid, block, 0, s,
                               static_cast<const uint32_t*>(a.words), static_cast<const _Float16*>(a.scales), layout, a.x, a.y,
                               a.y_dtype, a.rows, a.cols / (32 / kBits), a.word_pitch);
            break;
        default:
            hipLaunchKernelGGL((gemv_packed_kernel<kF, kBits, __bf16>), grid, block, 0, s,
                               static_cast<const uint32_t*>(a.words), static_cast<const __bf16*>(a.scales), layout, a.x, a.y,
                               a.y_dtype, a.rows, a.cols / (32 / kBits), a.word_pitch);
    }
    return hipGetLastError();
}

template <dev::Float kF>
hipError_t launch_general_bits(hipStream_t s, const GemvArgs& a, const dev::ScalesLayout& layout) {
    switch (a.bits) {
        case 2: return launch_general<kF, 2>(s, a, layout);
        case 4: return launch_general<kF, 4>(s, a, layout);
        case 8: return launch_general<kF, 8>(s, a, layout);
        default: return hipErrorInvalidValue;
    }
}

constexpr int kStreamRows = 4, kStreamChunks = 4, kStreamMaxStrips = 16;

template <dev::Float kF>
hipError_t launch_stream(hipStream_t s, const GemvArgs& a) {
    const uint32_t blocks_per_row = a.cols / 32;
    const uint32_t strips = (blocks_per_row + 63) / 64;
    // Seven rows per wave, fewer where that would leave fewer than four waves per SIMD (256 compute units x 4
    // SIMDs).  Measured on MI355X with 4096 / 8192 / 16384 / 32768 waves per launch: weights [14336, 4096]
    // 11.5 / 11.7 / 13.4 / 19.4 us, [28672, 8192] 34.5 / 31.7 / 30.0 / 31.5 us: about seven rows per wave in
    // both, enough rows to pay for a wave's 64 bytes of x per lane and enough waves to even out their ends.
    const uint64_t row_strips = static_cast<uint64_t>(a.rows) * strips;
    uint32_t rows_per_group = static_cast<uint32_t>((row_strips + 4095) / 4096);
    if (rows_per_group < 1) rows_per_group = 1;
    if (rows_per_group > 7) rows_per_group = 7;
    const dim3 grid((a.rows + rows_per_group - 1) / rows_per_group), block(64 * strips);
    dev::GlobalScaleLayout<1, 32> scale_at;
    scale_at.stride_row = static_cast<uint32_t>(a.scale_stride_row);
    scale_at.stride_col = static_cast<uint32_t>(a.scale_stride_col);
    hipLaunchKernelGGL((gemv_w4_b32_kernel<kF, float, kStreamRows, kStreamChunks, kStreamMaxStrips>), grid, block, 0, s,
                       static_cast<const uint32_t*>(a.words), static_cast<const float*>(a.scales), a.x, a.y, a.y_dtype, a.rows,
                       blocks_per_row, rows_per_group, a.word_pitch, scale_at);
    return hipGetLastError();
}

}  // namespace

bool gemv_streams(const GemvArgs& a) {
    return a.dtype != CQ_F32 && a.bits == 4 && a.block_rows == 1 && a.block_cols == 32 && a.param_dtype == CQ_F32 &&
           a.cols % 32 == 0 && a.cols / 32 <= 64u * kStreamMaxStrips && a.word_pitch % 4 == 0 && a.x_aligned16 &&
           a.words_aligned16 && a.rows < (1u << 26) && static_cast<uint64_t>(a.rows) * a.scale_stride_row < (1ull << 32) &&
           (a.cols / 32) * a.scale_stride_col < (1ull << 32);
}

hipError_t launch_gemv_quantized(hipStream_t s, const GemvArgs& a) {
    if (a.rows == 0 || a.cols == 0) return hipSuccess;
    if (gemv_streams(a)) return a.dtype == CQ_BF16 ? launch_stream<dev::Float::BF16>(s, a) : launch_stream<dev::Float::F16>(s, a);
    // the N-D layout of the [rows, cols] matrix, as the reference's scales_layout builds it
    dev::ScalesLayout layout;
    if (a.block_rows != 0) {
        const uint64_t vshape[2] = {a.rows, a.cols / (32u / a.bits)}, strides[2] = {a.scale_stride_row, a.scale_stride_col};
        const uint8_t block[2] = {static_cast<uint8_t>(a.block_rows), static_cast<uint8_t>(a.block_cols)};
        layout = dev::scales_layout(vshape, 2, 32u / a.bits, strides, block, 2);
    }
    switch (a.dtype) {
        case CQ_F32: return launch_general_bits<dev::Float::F32>(s, a, layout);
        case CQ_F16: return launch_general_bits<dev::Float::F16>(s, a, layout);
        case CQ_BF16: return launch_general_bits<dev::Float::BF16>(s, a, layout);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace cq
