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

// ---- streaming kernel: 16-bit float types, blocks along the row ---------------------------------------
// A lane's unit is one 16-byte load of codes: four words, 64 values of 2 bits, 32 of 4 or 16 of 8, under one scale
// (f32, f16 or bf16; blocks of 1, 2, 4, ... units along the row and any number of rows, or one scale for the
// tensor: a shift of 31 and strides of 0).  A wave owns kRows rows and walks along them, strip by strip (64 units, a lane
// per unit), so every wave of a launch does the same work whatever the number of strips, and the row sums never
// leave the wave: six DPP additions per row at its end, no exchange between waves, no barrier after the first.
// (With a wave per strip and the strips of a row in one workgroup, 5 to 8 strips all took the time of 8: the
// waves of a workgroup go round the four SIMDs from the first one, and the arithmetic, which is what bounds this
// kernel, piled up there.)  x is staged in LDS once per workgroup, with zeros behind its end up to a whole strip,
// so idle lanes add nothing, and read from there, a unit's values per lane and strip.  The loads of strip
// s + kDepth are issued as soon as strip s has been worked on; past the wave's last strip they fetch one uniform
// address instead of nothing, so that the number of loads in flight is the same in every iteration and the
// compiler can count its waits.  Per 4-bit value: half a byte-to-float conversion and one FMA
// (dequantize_symmetric_packed_value_pairs), half a v_cvt_pk, half a v_dot2.
// kCode: 2, 4 or 8 for fields of that many bits in the U32 store (and the i8 bytes of the native store, which are
// the same bits), or one of the native encodings below.
constexpr int kCodeE4M3 = 100, kCodeE5M2 = 101, kCodeE2M1x2 = 102;

// kVectors: 1, or room for that many right-hand vectors at once (x is then `vectors` <= kVectors rows of
// x_stride elements, y as many rows of y_stride): every dequantized pair is used kVectors times out of its
// registers, so a batch of vectors costs the weights' traffic and their dequantization once.
// kSegment (several vectors, or rows too long for the LDS): strips of x staged at a time; the workgroup meets at a
// barrier and stages the next ones when its waves have worked through them (they all do the same work, so nobody
// waits long).  0: all of x at once.
template <dev::Float kF, class FS, int kCode, int kRows, int kWaves, int kDepth, int kVectors, int kSegment = 0>
__global__ __launch_bounds__(64 * kWaves) void gemv_stream_kernel(
    const uint32_t* __restrict__ words, const FS* __restrict__ scales, const void* __restrict__ x, void* __restrict__ y,
    int y_dtype, uint32_t rows, uint32_t units_per_row, uint32_t units_per_block_log2, uint32_t block_rows,
    uint64_t word_pitch, uint32_t scale_stride_row, uint32_t scale_stride_col, uint32_t vectors, uint32_t x_stride,
    uint32_t y_stride) {
    constexpr bool kPacked = kCode <= 8;
    constexpr int kBits = kPacked ? kCode : 8;      // (of the packed fields)
    constexpr uint32_t kVals = kPacked ? 128 / kBits : (kCode == kCodeE2M1x2 ? 32 : 16);  // values of a unit
    constexpr bool kWide32 = kF == dev::Float::F32;  // x in f32: no pairs, the plain dequantization and one FMA per value
    constexpr uint32_t kPairs = kVals / 2;          // ... as packed pairs of x
    constexpr uint32_t kVecs = kWide32 ? kVals / 4 : kPairs / 4;  // ... as 16-byte pieces of x
    constexpr uint32_t kWordVals = kVals / 4;       // values out of one word
    static_assert(!kWide32 || kVectors == 1, "several vectors at once: 16-bit float types");
    constexpr uint32_t kWordPairs = kVals / 8;      // pairs out of one word
    constexpr dev::Native kNative = kCode == kCodeE4M3 ? dev::Native::E4M3
                                    : kCode == kCodeE5M2 ? dev::Native::E5M2 : dev::Native::E2M1x2;
    extern __shared__ u32x4 xs[];  // x, kVecs pieces per unit, whole strips; vector after vector
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t strips = (units_per_row + 63u) / 64u;
    constexpr bool kSegmented = kSegment > 0;
    constexpr uint32_t kSegmentOr1 = kSegment > 0 ? kSegment : 1;
    static_assert(kVectors == 1 || kSegmented, "several vectors are staged in segments");
    static_assert(kSegment % kDepth == 0, "segments of whole rounds of the ring");
    const uint32_t xs_vector = (kSegmented ? min(static_cast<uint32_t>(kSegment), strips) : strips) * 64u * kVecs;  // pieces of one staged vector
    // strips [first, first + xs_vector / (64 * kVecs)) of every vector into LDS, zeros behind the end of x
    const auto stage = [&](uint32_t first) {
#pragma unroll
        for (int v = 0; v < kVectors; v++) {
            const u32x4* xv = reinterpret_cast<const u32x4*>(static_cast<const char*>(x) + static_cast<uint64_t>(v) * x_stride * (kWide32 ? 4u : 2u));
            for (uint32_t i = threadIdx.x; i < xs_vector; i += blockDim.x) {
                const uint32_t at = first * 64u * kVecs + i;
                xs[v * xs_vector + i] = (static_cast<uint32_t>(v) < vectors && at < units_per_row * kVecs) ? xv[at] : u32x4{0, 0, 0, 0};
            }
        }
    };
    if constexpr (!kSegmented) {
        stage(0);
        __syncthreads();
    }
    // (segmented: a wave past the last row goes through the motions on the last row, for the barriers' sake)
    const bool idle = (blockIdx.x * kWaves + wave) * kRows >= rows;
    if (!kSegmented && idle) return;
    const uint32_t row0 = idle ? rows - 1u : (blockIdx.x * kWaves + wave) * kRows;
    const uint32_t nrows = min(static_cast<uint32_t>(kRows), rows - row0);

    struct Chunk {
        u32x4 w[kRows];
        FS s[kRows];
    };
    // the rows' first bytes, wave-uniform; rows past the end are the last row again
    const char* wrow[kRows];
    const char* srow[kRows];
#pragma unroll
    for (int k = 0; k < kRows; k++) {
        const uint32_t r = row0 + min(static_cast<uint32_t>(k), nrows - 1u);
        wrow[k] = reinterpret_cast<const char*>(words + static_cast<uint64_t>(r) * word_pitch);
        srow[k] = reinterpret_cast<const char*>(scales + static_cast<uint64_t>(r / block_rows) * scale_stride_row);
    }
    const uint32_t scale_step = scale_stride_col * static_cast<uint32_t>(sizeof(FS));
    const auto load = [&](Chunk& c, uint32_t strip) {
        const bool real = strip < strips;  // wave-uniform
        const uint32_t u = min(strip * 64u + lane, units_per_row - 1u);  // idle lanes re-read the row's last unit
        const uint32_t woff = real ? u * 16u : 0u, soff = real ? (u >> units_per_block_log2) * scale_step : 0u;
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            c.w[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[k] + woff));
            c.s[k] = __builtin_nontemporal_load(reinterpret_cast<const FS*>(srow[k] + soff));
        }
        __builtin_amdgcn_sched_barrier(0);  // loads stay where they are written: kDepth strips ahead of the arithmetic
    };
    // One row's share of this lane, the plain way (rolled loops, operands read again).  Only lanes whose scale
    // is not tame come here.
    const auto plain_row = [&](const char* words_of_row, const char* scales_of_row, uint32_t strip, uint32_t v) {
        if constexpr (kWide32) {
            return 0.0f;  // (f32 x: the main path is the plain one)
        } else {
            const uint32_t u = strip * 64u + lane;
            if (!kPacked || u >= units_per_row || v >= vectors) return 0.0f;
            const uint32_t* wr = reinterpret_cast<const uint32_t*>(words_of_row) + u * 4u;
            const FS scale = *reinterpret_cast<const FS*>(scales_of_row + (u >> units_per_block_log2) * scale_step);
            const typename Elem<kF>::T* xr = static_cast<const typename Elem<kF>::T*>(x) + static_cast<uint64_t>(v) * x_stride + u * kVals;
            float a = 0.0f;
    #pragma unroll 1
            for (int j = 0; j < 4; j++) {
                float v[2 * kWordPairs];
                dev::dequantize_symmetric_packed_value<kF, kBits>(wr[j], scale, v);
    #pragma unroll
                for (uint32_t i = 0; i < 2 * kWordPairs; i += 2) {
                    const uint32_t xpair =
                        static_cast<uint32_t>(__builtin_bit_cast(uint16_t, xr[2 * kWordPairs * j + i])) |
                        static_cast<uint32_t>(__builtin_bit_cast(uint16_t, xr[2 * kWordPairs * j + i + 1])) << 16;
                    a = dot2<kF>(dev::pack_pair<kF>(v[i], v[i + 1]), xpair, a);
                }
            }
            return a;
        }
    };
    float acc[kRows * kVectors];
#pragma unroll
    for (int k = 0; k < kRows * kVectors; k++) acc[k] = 0.0f;
    // Lanes past the end of a row's last strip hold the row's last unit again (see `load`) against zeros of x: their
    // share is dropped, not added, because an infinite or NaN scale in that unit would turn the zeros into NaN.
    const auto lane_holds = [&](uint32_t strip) { return strip * 64u + lane < units_per_row; };
    // several vectors: the pairs of the chunk's rows once, then vector after vector against them
    const auto work_vectors = [&](const Chunk& c, uint32_t strip) {
        if constexpr (kVectors > 1) {
            uint32_t pairs[kRows][kPairs];
            bool tame = true;
    #pragma unroll
            for (int k = 0; k < kRows; k++) {
    #pragma unroll
                for (int j = 0; j < 4; j++) {
                    if constexpr (kPacked)
                        dev::dequantize_symmetric_packed_value_pairs_tame<kF, kBits>(c.w[k][j], c.s[k], &pairs[k][kWordPairs * j]);
                    else
                        dev::dequantize_symmetric_native_value_pairs<kF, kNative>(c.w[k][j], c.s[k], &pairs[k][kWordPairs * j]);
                }
                if constexpr (kPacked) tame = tame && dev::pairs_scale_is_tame<kF>(c.s[k]);
            }
            float part[kRows * kVectors];
    #pragma unroll
            for (int v = 0; v < kVectors; v++) {
                uint32_t xp[kPairs];
    #pragma unroll
                for (uint32_t j = 0; j < kVecs; j++) {
                    const u32x4 t = xs[v * xs_vector + ((strip % kSegmentOr1) * 64u + lane) * kVecs + j];
                    xp[4 * j] = t[0], xp[4 * j + 1] = t[1], xp[4 * j + 2] = t[2], xp[4 * j + 3] = t[3];
                }
    #pragma unroll
                for (int k = 0; k < kRows; k++) {
                    float a = 0.0f;
    #pragma unroll
                    for (uint32_t i = 0; i < kPairs; i++) a = dot2<kF>(pairs[k][i], xp[i], a);
                    part[k * kVectors + v] = a;
                }
            }
            // lanes whose scale is not tame: the plain way, one (row, vector) at a time in a rolled loop (one copy of
            // the code; unrolled, it took the compiler minutes)
            if (kPacked && __builtin_amdgcn_ballot_w64(!tame) != 0) {
                uint32_t plain_rows = 0;  // per lane: bit k set, row k's scale is not tame
    #pragma unroll
                for (int k = 0; k < kRows; k++) plain_rows |= dev::pairs_scale_is_tame<kF>(c.s[k]) ? 0u : 1u << k;
    #pragma unroll 1
                for (int kv = 0; kv < kRows * kVectors; kv++) {
                    const int k = kv / kVectors;
                    const char* wr = wrow[0];
                    const char* sr = srow[0];
    #pragma unroll
                    for (int t = 1; t < kRows; t++) {
                        if (k == t) wr = wrow[t], sr = srow[t];
                    }
                    if ((plain_rows >> k) & 1u) {
                        const float r = plain_row(wr, sr, strip, static_cast<uint32_t>(kv % kVectors));
    #pragma unroll
                        for (int t = 0; t < kRows * kVectors; t++) part[t] = t == kv ? r : part[t];
                    }
                }
            }
    #pragma unroll
            for (int k = 0; k < kRows * kVectors; k++) acc[k] += lane_holds(strip) ? part[k] : 0.0f;
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    const auto work = [&](const Chunk& c, uint32_t strip) {
        if constexpr (kWide32) {
            // this lane's values of x
            float xf[kVals];
#pragma unroll
            for (uint32_t j = 0; j < kVecs; j++) {
                const u32x4 t = xs[((kSegmented ? strip % kSegmentOr1 : strip) * 64u + lane) * kVecs + j];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t bits = t[i];  // (a bit cast of the element expression itself reads element 0)
                    xf[4 * j + i] = __builtin_bit_cast(float, bits);
                }
            }
#pragma unroll
            for (int k = 0; k < kRows; k++) {
                float a = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float v[kWordVals];
                    if constexpr (kPacked)
                        dev::dequantize_symmetric_packed_value<kF, kBits>(c.w[k][j], c.s[k], v);
                    else
                        dev::dequantize_symmetric_native_value<kF, kNative>(c.w[k][j], c.s[k], v);
#pragma unroll
                    for (uint32_t i = 0; i < kWordVals; i++) a = __builtin_fmaf(v[i], xf[kWordVals * j + i], a);
                }
                acc[k] += lane_holds(strip) ? a : 0.0f;
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
            if constexpr (kVectors > 1) {
                work_vectors(c, strip);
                return;
            }
            // this lane's values of x, as pairs
            uint32_t xp[kPairs];
    #pragma unroll
            for (uint32_t j = 0; j < kVecs; j++) {
                const u32x4 v = xs[((kSegmented ? strip % kSegmentOr1 : strip) * 64u + lane) * kVecs + j];
                xp[4 * j] = v[0], xp[4 * j + 1] = v[1], xp[4 * j + 2] = v[2], xp[4 * j + 3] = v[3];
            }
            float part[kRows];
            if constexpr (kPacked) {
                bool tame = true;
    #pragma unroll
                for (int k = 0; k < kRows; k++) {
                    float a = 0.0f;
    #pragma unroll
                    for (int j = 0; j < 4; j++) {
                        uint32_t pairs[kWordPairs];
                        dev::dequantize_symmetric_packed_value_pairs_tame<kF, kBits>(c.w[k][j], c.s[k], pairs);
    #pragma unroll
                        for (uint32_t i = 0; i < kWordPairs; i++) a = dot2<kF>(pairs[i], xp[kWordPairs * j + i], a);
                    }
                    part[k] = a;
                    tame = tame && dev::pairs_scale_is_tame<kF>(c.s[k]);
                }
                // ordinary scales are all tame: one wave-uniform test per chunk, then straight on
                if (__builtin_amdgcn_ballot_w64(!tame) != 0) {
    #pragma unroll
                    for (int k = 0; k < kRows; k++)
                        if (!dev::pairs_scale_is_tame<kF>(c.s[k])) part[k] = plain_row(wrow[k], srow[k], strip, 0);
                }
            } else {
                // native encodings: the pairs are the plain arithmetic, every scale goes the same way
    #pragma unroll
                for (int k = 0; k < kRows; k++) {
                    float a = 0.0f;
    #pragma unroll
                    for (int j = 0; j < 4; j++) {
                        uint32_t pairs[kWordPairs];
                        dev::dequantize_symmetric_native_value_pairs<kF, kNative>(c.w[k][j], c.s[k], pairs);
    #pragma unroll
                        for (uint32_t i = 0; i < kWordPairs; i++) a = dot2<kF>(pairs[i], xp[kWordPairs * j + i], a);
                    }
                    part[k] = a;
                }
            }
    #pragma unroll
            for (int k = 0; k < kRows; k++) acc[k] += lane_holds(strip) ? part[k] : 0.0f;
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    Chunk c[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; d++) load(c[d], d);
    for (uint32_t strip = 0; strip < strips; strip += kDepth) {
        if constexpr (kSegmented) {
            if (strip % kSegmentOr1 == 0) {
                if (strip != 0) __syncthreads();  // everybody has read the strips that are about to be replaced
                stage(strip);
                __syncthreads();
            }
        }
#pragma unroll
        for (int d = 0; d < kDepth; d++) {
            if (d == 0 || strip + d < strips) work(c[d], strip + d);
            load(c[d], strip + d + kDepth);
        }
    }
#pragma unroll
    for (int k = 0; k < kRows * kVectors; k++) acc[k] = wave_sum_to_lane63(acc[k]);
    if (lane == 63) {
#pragma unroll
        for (int k = 0; k < kRows; k++) {
#pragma unroll
            for (int v = 0; v < kVectors; v++)
                if (!idle && static_cast<uint32_t>(k) < nrows && static_cast<uint32_t>(v) < vectors)
                    store_y(y_dtype, y, static_cast<uint64_t>(v) * y_stride + row0 + k, acc[k * kVectors + v]);
        }
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

constexpr int kStreamRows = 2, kStreamDepth = 2;
[[maybe_unused]] constexpr uint32_t kStreamMaxColumns = 32768;  // x of that many columns fills 64 KiB of LDS

uint32_t log2_of(uint32_t v) {
    uint32_t l = 0;
    while ((1u << l) < v) l++;
    return l;
}

constexpr uint32_t values_per_unit(int code) { return code <= 8 ? 128 / code : (code == kCodeE2M1x2 ? 32 : 16); }

// LDS for x: whole strips, 2 bytes per value, times the vectors staged at once
uint32_t stream_lds_bytes(const GemvArgs& a, uint32_t vectors) {
    const uint32_t vals = 128 / a.bits;
    return (a.cols / vals + 63) / 64 * 64 * vals * (a.dtype == CQ_F32 ? 4 : 2) * vectors;
}

template <dev::Float kF, class FS, int kBits, int kWaves, int kVectors, int kRows = kStreamRows, int kSegment = 0>
void launch_stream_waves(hipStream_t s, const GemvArgs& a) {
    constexpr uint32_t kVals = values_per_unit(kBits);
    const uint32_t units_per_row = a.cols / kVals;
    const dim3 grid((a.rows + kRows * kWaves - 1) / (kRows * kWaves)), block(64 * kWaves);
    const uint32_t strips = (units_per_row + 63) / 64;
    const uint32_t lds = kSegment > 0 ? (strips < kSegment ? strips : kSegment) * 64 * kVals * (kF == dev::Float::F32 ? 4 : 2) * kVectors
                                      : stream_lds_bytes(a, 1);
    hipLaunchKernelGGL((gemv_stream_kernel<kF, FS, kBits, kRows, kWaves, kStreamDepth, kVectors, kSegment>), grid, block,
                       lds, s, static_cast<const uint32_t*>(a.words),
                       static_cast<const FS*>(a.scales), a.x, a.y, a.y_dtype, a.rows, units_per_row,
                       a.block_rows == 0 ? 31u : log2_of(a.block_cols / kVals), a.block_rows == 0 ? 1u : a.block_rows,
                       a.word_pitch, static_cast<uint32_t>(a.scale_stride_row), static_cast<uint32_t>(a.scale_stride_col),
                       a.vectors, static_cast<uint32_t>(a.x_stride), static_cast<uint32_t>(a.y_stride));
}

// Two rows per wave, two strips in flight, four waves (eight rows) per workgroup; eight waves from 16384 columns
// on, where the 32 KiB and more of x that every workgroup stages weigh more than the smaller workgroup gains.
// Measured on MI355X (rows / waves / strips in flight; 4-bit weights [14336, 4096], [28672, 8192], [4096, 11008],
// [8192, 28672]): 2 / 4 / 2 10.1, 31.3, 9.5, 33.5 us; 2 / 8 / 2 11.2, 33.1, 9.0, 28.9 us; 2 / 4 / 3 10.3, 33.0,
// 10.1, 33.4 us; 4 / 4 / 2 11.8, 36.5, 10.3, 32.6 us; 1 / 4 / 4 11.4, 34.0, 10.1, 43.3 us; 3 / 4 / 2 10.8, 31.2,
// 11.7, 34.5 us.
// Right-hand vectors at once, and the waves of a workgroup that shares their x, rows per wave.  Measured on MI355X,
// four vectors on 4-bit [28672, 8192] / [14336, 4096] / [4096, 8192] and e4m3 bytes [28672, 8192] (waves / rows):
// 8 / 2 56.8, 19.3, 12.2, 57.1 us; 16 / 2 63.5, 19.6, 15.3, 67.9 us; 8 / 4 60.0, 20.1, 17.0, 71.7 us; 4 / 2 79.0,
// 19.6, 13.0, 82.2 us; 16 / 4 68.6, 22.5, 29.6, 68.3 us.
// Strips of x staged at a time (64 KiB of LDS for four vectors of 4-bit units): 4; with 2, [28672, 8192] took 63.0
// instead of 57.4 us (e4m3 bytes 72.4 instead of 60.5 us), with 8 (half as many 4-bit workgroups per compute
// unit) 83.3 us.
constexpr int kBatch = 4, kBatchWaves = 8, kBatchRows = 2, kBatchSegment = 4;
constexpr bool batches(int code) { return code != 2; }  // (64 values per unit: their pairs alone would fill the registers)

constexpr int kWideSegment = 16;  // strips of x at a time where a row has more than kStreamMaxColumns values

template <dev::Float kF, class FS, int kBits, bool kBatched>
void launch_stream_bits(hipStream_t s, const GemvArgs& a) {
    if constexpr (kBatched) {
        if (a.vectors == 1)  // one right-hand side, rows too long for the LDS
            launch_stream_waves<kF, FS, kBits, 8, 1, kStreamRows,
                                kWideSegment * int(values_per_unit(4)) / int(values_per_unit(kBits)) / (kF == dev::Float::F32 ? 2 : 1)>(s, a);
        else if constexpr (batches(kBits) && kF != dev::Float::F32)
            launch_stream_waves<kF, FS, kBits, kBatchWaves, kBatch, kBatchRows, kBatchSegment>(s, a);
    } else if (a.cols >= 16384) {
        launch_stream_waves<kF, FS, kBits, 8, 1>(s, a);
    } else {
        launch_stream_waves<kF, FS, kBits, 4, 1>(s, a);
    }
}

template <dev::Float kF, class FS, bool kBatched>
void launch_stream_scales(hipStream_t s, const GemvArgs& a) {
    if (a.native == 1)
        launch_stream_bits<kF, FS, kCodeE4M3, kBatched>(s, a);
    else if (a.native == 2)
        launch_stream_bits<kF, FS, kCodeE5M2, kBatched>(s, a);
    else if (a.native == 3)
        launch_stream_bits<kF, FS, kCodeE2M1x2, kBatched>(s, a);
    else if (a.bits == 4)
        launch_stream_bits<kF, FS, 4, kBatched>(s, a);
    else if (a.bits == 8)
        launch_stream_bits<kF, FS, 8, kBatched>(s, a);
    else
        launch_stream_bits<kF, FS, 2, kBatched>(s, a);
}

template <class FS, bool kBatched>
hipError_t launch_stream_floats(hipStream_t s, const GemvArgs& a) {
    if (a.dtype == CQ_BF16)
        launch_stream_scales<dev::Float::BF16, FS, kBatched>(s, a);
    else
        launch_stream_scales<dev::Float::F16, FS, kBatched>(s, a);
    return hipGetLastError();
}

}  // namespace

// The streaming kernels sit in three objects, so that a process loads the code of the kind it uses (the first launch
// out of an object loads all of it): one right-hand side with f32 scales, with f16 / bf16 scales, several at once
// (and rows too long for the LDS), x in f32.
// CQ_GEMV_PART names the one being compiled; without it everything lands in one object.
#if !defined(CQ_GEMV_PART) || CQ_GEMV_PART == 0
hipError_t gemv_stream_f32_scales(hipStream_t s, const GemvArgs& a) { return launch_stream_floats<float, false>(s, a); }
#endif
#if !defined(CQ_GEMV_PART) || CQ_GEMV_PART == 1
hipError_t gemv_stream_16bit_scales(hipStream_t s, const GemvArgs& a) {
    return a.param_dtype == CQ_F16 ? launch_stream_floats<_Float16, false>(s, a) : launch_stream_floats<__bf16, false>(s, a);
}
#endif
#if !defined(CQ_GEMV_PART) || CQ_GEMV_PART == 2
hipError_t gemv_stream_batched(hipStream_t s, const GemvArgs& a) {
    switch (a.param_dtype) {
        case CQ_F32: return launch_stream_floats<float, true>(s, a);
        case CQ_F16: return launch_stream_floats<_Float16, true>(s, a);
        default: return launch_stream_floats<__bf16, true>(s, a);
    }
}
#endif

#if !defined(CQ_GEMV_PART) || CQ_GEMV_PART == 3
// x in f32 (f32 scales): the plain dequantization and one FMA per value
hipError_t gemv_stream_f32_x(hipStream_t s, const GemvArgs& a) {
    if (a.cols > kStreamMaxColumns / 2)
        launch_stream_scales<dev::Float::F32, float, true>(s, a);
    else
        launch_stream_scales<dev::Float::F32, float, false>(s, a);
    return hipGetLastError();
}
#endif

#if !defined(CQ_GEMV_PART) || CQ_GEMV_PART == 0
bool gemv_streams(const GemvArgs& a) {
    if ((a.bits != 2 && a.bits != 4 && a.bits != 8) || (a.dtype == CQ_F32 && a.param_dtype != CQ_F32)) return false;
    const uint32_t vals = 128 / a.bits;  // values of a 16-byte unit (native encodings come with their bits)
    if (a.block_rows != 0) {             // blocks: whole units along the row, a power of two of them
        const uint32_t units_per_block = a.block_cols / vals;
        if (a.block_cols % vals != 0 || (units_per_block & (units_per_block - 1)) != 0 || a.cols % a.block_cols != 0 ||
            a.scale_stride_row >= (1ull << 32) || (a.cols / a.block_cols) * a.scale_stride_col >= (1ull << 29))
            return false;
    }
    if (a.x_stride >= (1ull << 32) || a.y_stride >= (1ull << 32)) return false;  // the kernels take them as 32-bit numbers
    return a.cols % vals == 0 && a.cols < (1u << 26) && a.word_pitch % 4 == 0 && a.x_aligned16 && a.words_aligned16;
}

namespace {

hipError_t launch_one(hipStream_t s, const GemvArgs& a) {
    if (gemv_mfma_takes(a)) return gemv_mfma(s, a);  // two to four vectors of the common 4-bit layout: matrix cores
    if (gemv_streams(a)) {
        if (a.dtype == CQ_F32) return gemv_stream_f32_x(s, a);
        if (a.vectors > 1 || a.cols > kStreamMaxColumns) return gemv_stream_batched(s, a);
        return a.param_dtype == CQ_F32 ? gemv_stream_f32_scales(s, a) : gemv_stream_16bit_scales(s, a);
    }
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

uint32_t dtype_bytes(int dtype) { return dtype == CQ_F32 ? 4u : 2u; }

}  // namespace

// How many of the remaining vectors the next launch takes: up to four at once where the streaming kernel applies
// (all but the 2-bit fields) and every one of them starts on a 16-byte boundary; else one.
uint32_t gemv_vectors_per_launch(const GemvArgs& a, uint32_t remaining) {
    if (remaining < 2 || !gemv_streams(a) || (a.x_stride * 2) % 16 != 0 || a.bits == 2 || a.dtype == CQ_F32) return 1;
    return remaining < kBatch ? remaining : kBatch;
}

// an empty sum: every y is zero
__global__ void gemv_zero_kernel(void* y, int y_dtype, uint32_t rows, uint32_t vectors, uint64_t y_stride) {
    const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    for (uint32_t v = 0; v < vectors; v++) store_y(y_dtype, y, static_cast<uint64_t>(v) * y_stride + r, 0.0f);
}

hipError_t launch_gemv_quantized(hipStream_t s, const GemvArgs& a) {
    if (a.rows == 0) return hipSuccess;
    if (a.cols == 0) {
        hipLaunchKernelGGL(gemv_zero_kernel, dim3((a.rows + 255) / 256), dim3(256), 0, s, a.y, a.y_dtype, a.rows, a.vectors, a.y_stride);
        return hipGetLastError();
    }
    for (uint32_t v = 0; v < a.vectors;) {
        GemvArgs b = a;
        b.x = static_cast<const char*>(a.x) + static_cast<uint64_t>(v) * a.x_stride * dtype_bytes(a.dtype);
        b.y = static_cast<char*>(a.y) + static_cast<uint64_t>(v) * a.y_stride * dtype_bytes(a.y_dtype);
        b.x_aligned16 = (reinterpret_cast<uintptr_t>(b.x) & 15u) == 0;
        b.vectors = gemv_vectors_per_launch(b, a.vectors - v);
        const hipError_t e = launch_one(s, b);
        if (e != hipSuccess) return e;
        v += b.vectors;
    }
    return hipSuccess;
}

#endif  // part 0

}  // namespace cq
