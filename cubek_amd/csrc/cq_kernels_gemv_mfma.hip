// y = dequantize(W) * x on the matrix cores, for 4-bit codes in the U32 store on blocks of 32 values with f32 scales and
// x in bf16 / f16: the layouts of the quantized-input arm of the reference's matmul
// (crates/cubek-matmul/src/base.rs:309-317; scale lookup components/global/memory/layout.rs:371-455) for two to four
// right-hand columns at once (one column stays with the streaming kernel, which is faster there: 31 us against 34 us on
// [28672, 8192]; four columns take 36 us here against 56 us there).  Every weight enters the product as cq_dequantize would store it, F(F(scale) * F(code))
// (crates/cubek-quant/src/dequantize.rs:20-79, through include/cubek_quant_device.hpp); products accumulate in f32.
//
// The weights want to be read as whole rows, 4 KiB and more at a stretch (bands of 512 bytes across 16 rows reach
// 57 % of the HBM peak on [28672, 8192], whole rows 78 %), and a 16 x 16 x 32 matrix instruction wants, in lane
// (i, g) = (lane % 16, lane / 16), eight consecutive values of its row i.  Both hold when the 16 "rows" of the
// instruction are 16 segments of 512 values: kQ consecutive segments of each of 16 / kQ rows.  Segment q of a row
// meets segment q of x, so the instruction's 16 columns are the kQ segments of x (times the right-hand vectors:
// kQ * vectors <= 16), and of its 16 x 16 results those with the same segment on both sides are kept: 1 / kQ of
// the arithmetic is of use, which the matrix cores have to spare.
//
// The codes go from global memory straight to LDS (global_load_lds_dwordx4: no registers, 1 KiB per instruction)
// and the lanes read their 16-byte units (32 values, one scale) back in the order the instruction wants.  Which
// lane loads which 16 bytes of a run is free, so the units of segment i are rotated by i places on their way in,
// and the 16 lanes of a read, which want the same unit of 16 segments, fall on 16 different groups of banks.  The
// scales (one instruction per step) and x (once per workgroup and stage of 512 * kQ values) come the same way,
// rotated likewise.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/cubek_quant_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

namespace dev = cubek_quant::device;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4a __attribute__((ext_vector_type(4), may_alias));
typedef float f32a __attribute__((may_alias));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kMfmaWaves = 4;
constexpr uint32_t kCodeBytes = 16 * 16 * 16;  // 16 segments of 16 units
constexpr uint32_t kScaleBytes = 16 * 16 * 4;
constexpr uint32_t kStepBytes = kCodeBytes + kScaleBytes;

constexpr uint32_t mfma_lds_bytes(int q, int vectors) {
    return static_cast<uint32_t>(vectors) * 1024u * static_cast<uint32_t>(q) + kMfmaWaves * kStepBytes;
}

template <dev::Float kF>
__device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    if constexpr (kF == dev::Float::BF16) {
        typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    } else {
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
}

#define CQ_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// kQ segments of 16 / kQ rows per step; a wave owns kRowsPerWave = max(4, 16 / kQ) rows, a workgroup four times that.
template <dev::Float kF, int kQ, int kVectors>
__global__ __launch_bounds__(64 * kMfmaWaves) void gemv_mfma_kernel(const char* __restrict__ words, const char* __restrict__ scales,
                                                                    const char* __restrict__ x, void* __restrict__ y, int y_dtype,
                                                                    uint32_t rows, uint32_t units_per_row, uint64_t row_bytes,
                                                                    uint64_t scale_row_bytes, uint32_t vectors, uint64_t x_stride_bytes,
                                                                    uint64_t y_stride) {
    static_assert(kQ == 1 || kQ == 2 || kQ == 4 || kQ == 8 || kQ == 16, "segments per row and step");
    static_assert(kVectors == 1 || kVectors == 2 || kVectors == 4, "vectors held at once");
    static_assert(kQ * kVectors <= 16, "the instruction has 16 columns");
    constexpr uint32_t kR = 16 / kQ;                     // rows of a step
    constexpr uint32_t kRowsPerWave = kR < 4 ? 4 : kR;
    constexpr uint32_t kBlocks = kRowsPerWave / kR;      // steps of a wave per stage
    constexpr uint32_t kStageUnits = 16 * kQ;            // units of a row per stage
    constexpr uint32_t kXBytes = 1024 * kQ;              // one vector's values of a stage
    extern __shared__ u32x4 lds[];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char* const x_img = reinterpret_cast<char*>(lds);
    char* const code_img = x_img + kVectors * kXBytes + wave * kStepBytes;  // wave-uniform
    char* const scale_img = code_img + kCodeBytes;
    const uint32_t row0 = (blockIdx.x * kMfmaWaves + wave) * kRowsPerWave;
    const uint32_t stages = (units_per_row + kStageUnits - 1) / kStageUnits;
    const uint32_t i = lane & 15u, g = lane >> 4;        // this lane's segment and unit of four in the instruction
    const uint32_t seg_q = i % kQ;

    f32x4 acc[kBlocks];
#pragma unroll
    for (uint32_t b = 0; b < kBlocks; b++) acc[b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // column i of the instruction: segment i % kQ of vector i / kQ (columns past the vectors repeat earlier ones)
    const uint32_t col_v = (i / kQ) & static_cast<uint32_t>(kVectors - 1);
    const uint32_t col_rot = (seg_q + kQ * col_v) & 15u;
    const char* const x_mine = x_img + col_v * kXBytes + seg_q * 1024u;  // 64 pieces of eight values

    for (uint32_t stage = 0; stage < stages; stage++) {
        const uint32_t unit0 = stage * kStageUnits;
        const bool partial = unit0 + kStageUnits > units_per_row;  // wave-uniform
        // ---- x of this stage, every wave its share of the kQ * kVectors instructions
        if (stage != 0) __syncthreads();  // everybody has read the stage that is about to be replaced
#pragma unroll
        for (uint32_t m = 0; m < static_cast<uint32_t>(kQ * kVectors); m++) {
            if (m % kMfmaWaves != wave) continue;
            const uint32_t v = m / kQ, mm = m % kQ;
            if (v >= vectors) continue;
            // place pl of the vector's image holds piece (block b = pl / 16, (pl % 16 - rot) % 16), rot = segment + kQ * v
            const uint32_t pl = 64u * mm + lane, b = pl >> 4;
            const uint32_t rot = ((b >> 2) + kQ * v) & 15u;
            const uint32_t piece = min(unit0 * 4u + ((b << 4) | ((pl - rot) & 15u)), units_per_row * 4u - 1u);
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(x + v * x_stride_bytes + piece * 16u),
                                             CQ_LDS_PTR(x_img + v * kXBytes + mm * 1024u), 16, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

#pragma unroll
        for (uint32_t blk = 0; blk < kBlocks; blk++) {
            // ---- the step's codes: place p of segment s holds unit (p - s) % 16; instruction t brings segments 4t .. 4t+3
#pragma unroll
            for (uint32_t t = 0; t < 4; t++) {
                const uint32_t s = 4u * t + (lane >> 4);
                const uint32_t unit = min(unit0 + (s % kQ) * 16u + ((lane - s) & 15u), units_per_row - 1u);
                const uint32_t row = min(row0 + blk * kR + s / kQ, rows - 1u);
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(words + static_cast<uint64_t>(row) * row_bytes + unit * 16u),
                                                 CQ_LDS_PTR(code_img + t * 1024u), 16, 0, 2 /* nt */);
            }
            // ---- its scales: four pieces of four per segment; place p of segment s holds piece (p - s / 4) % 4
            {
                const uint32_t s = lane >> 2;
                const uint32_t piece = min(unit0 / 4u + (s % kQ) * 4u + ((lane - (s >> 2)) & 3u), units_per_row / 4u - 1u);
                const uint32_t row = min(row0 + blk * kR + s / kQ, rows - 1u);
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(scales + static_cast<uint64_t>(row) * scale_row_bytes + piece * 16u),
                                                 CQ_LDS_PTR(scale_img), 16, 0, 2 /* nt */);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

            u32x4 cw[4];
            float sc[4];
            bool tame = true;
#pragma unroll
            for (uint32_t grp = 0; grp < 4; grp++) {
                cw[grp] = *reinterpret_cast<const u32x4a*>(code_img + i * 256u + ((4u * grp + g + i) & 15u) * 16u);
                sc[grp] = *reinterpret_cast<const f32a*>(scale_img + i * 64u + ((grp + (i >> 2)) & 3u) * 16u + g * 4u);
                tame = tame && dev::pairs_scale_is_tame<kF>(sc[grp]);
            }
            const bool all_tame = __builtin_amdgcn_ballot_w64(!tame) == 0;  // wave-uniform; ordinary scales all are
            // the step's 16 instructions: with the short dequantization or the general one, with or without the mask
            // of a row's end (three copies of the code behind uniform branches)
            const auto work = [&](auto tame_tag, auto mask_tag) {
                constexpr bool kTame = decltype(tame_tag)::value, kMask = decltype(mask_tag)::value;
#pragma unroll
                for (uint32_t grp = 0; grp < 4; grp++) {
                    const bool past = kMask && unit0 + seg_q * 16u + 4u * grp + g >= units_per_row;
#pragma unroll
                    for (uint32_t j = 0; j < 4; j++) {
                        uint32_t pairs[4];
                        u32x4 b = *reinterpret_cast<const u32x4a*>(x_mine + (grp << 8) + ((4u * g + j + col_rot) & 15u) * 16u);
                        if constexpr (kTame)
                            dev::dequantize_symmetric_packed_value_pairs_tame<kF, 4>(cw[grp][j], sc[grp], pairs);
                        else
                            dev::dequantize_symmetric_packed_value_pairs<kF, 4>(cw[grp][j], sc[grp], pairs);
                        if (past) {  // past the end of the row: nothing, whatever the clamped loads brought
                            pairs[0] = pairs[1] = pairs[2] = pairs[3] = 0u;
                            b = u32x4{0, 0, 0, 0};
                        }
                        acc[blk] = mfma<kF>(u32x4{pairs[0], pairs[1], pairs[2], pairs[3]}, b, acc[blk]);
                    }
                }
            };
            if (all_tame && !partial)
                work(std::true_type{}, std::false_type{});
            else if (all_tame)
                work(std::true_type{}, std::true_type{});
            else
                work(std::false_type{}, std::true_type{});
        }
    }
    // acc[blk][r] = (segment 4 g + r of the step, column i): of use where both segments are the same one; a row's kQ
    // segments meet in LDS (the wave's own image; its reads are behind it: LDS takes a wave's accesses in order)
    float* const part = reinterpret_cast<float*>(code_img);
#pragma unroll
    for (uint32_t blk = 0; blk < kBlocks; blk++) {
#pragma unroll
        for (uint32_t r = 0; r < 4; r++) {
            const uint32_t s = 4u * g + r;  // segment of the step
            if (s % kQ == seg_q && i / kQ < vectors)
                part[((blk * kR + s / kQ) * kVectors + i / kQ) * kQ + seg_q] = acc[blk][r];
        }
    }
    if (lane < kRowsPerWave * kVectors) {
        const uint32_t r = lane / kVectors, v = lane % kVectors;
        float sum = 0.0f;
#pragma unroll
        for (uint32_t q = 0; q < static_cast<uint32_t>(kQ); q++) sum += part[lane * kQ + q];
        if (row0 + r < rows && v < vectors) {
            const uint64_t at = v * y_stride + row0 + r;
            if (y_dtype == CQ_F32)
                static_cast<float*>(y)[at] = sum;
            else if (y_dtype == CQ_F16)
                static_cast<_Float16*>(y)[at] = static_cast<_Float16>(sum);
            else
                static_cast<__bf16*>(y)[at] = static_cast<__bf16>(sum);
        }
    }
}

template <dev::Float kF, int kQ, int kVectors>
void launch_shape(hipStream_t s, const GemvArgs& a) {
    constexpr uint32_t kRowsPerWave = 16 / kQ < 4 ? 4 : 16 / kQ;
    const uint32_t rows_per_group = kRowsPerWave * kMfmaWaves;
    hipLaunchKernelGGL((gemv_mfma_kernel<kF, kQ, kVectors>), dim3((a.rows + rows_per_group - 1) / rows_per_group), dim3(64 * kMfmaWaves),
                       mfma_lds_bytes(kQ, kVectors), s, static_cast<const char*>(a.words), static_cast<const char*>(a.scales),
                       static_cast<const char*>(a.x), a.y, a.y_dtype, a.rows, a.cols / 32, a.word_pitch * 4, a.scale_stride_row * 4,
                       a.vectors, a.x_stride * 2, a.y_stride);
}

// Two vectors: runs of 4096 values of a row per step where the row is a whole number of them (or of nothing shorter);
// three and four: runs of 2048.
template <dev::Float kF>
void launch_float(hipStream_t s, const GemvArgs& a) {
    if (a.vectors == 2) {
        if (a.cols % 4096 == 0 || a.cols % 2048 != 0)
            launch_shape<kF, 8, 2>(s, a);
        else
            launch_shape<kF, 4, 2>(s, a);
    } else {
        launch_shape<kF, 4, 4>(s, a);
    }
}

}  // namespace

// 4-bit fields in u32 words, one f32 scale per 32 values stored one after the other along the row, x in a 16-bit
// type, rows of whole groups of four units, everything the 16-byte loads touch on 16-byte boundaries.
bool gemv_mfma_takes(const GemvArgs& a) {
    if (a.native != 0 || a.bits != 4 || a.param_dtype != CQ_F32 || a.dtype == CQ_F32) return false;
    if (a.block_rows != 1 || a.block_cols != 32 || a.scale_stride_col != 1) return false;
    if (a.cols % 128 != 0 || a.cols < 4096 || a.cols >= (1u << 26) || a.rows >= (1u << 31)) return false;
    if (a.word_pitch % 4 != 0 || a.scale_stride_row % 4 != 0 || !a.x_aligned16 || !a.words_aligned16) return false;
    if ((reinterpret_cast<uintptr_t>(a.scales) & 15u) != 0) return false;
    if (a.vectors > 1 && (a.x_stride * 2) % 16 != 0) return false;
    return a.vectors >= 2 && a.vectors <= 4;
}

hipError_t gemv_mfma(hipStream_t s, const GemvArgs& a) {
    if (a.dtype == CQ_BF16)
        launch_float<dev::Float::BF16>(s, a);
    else
        launch_float<dev::Float::F16>(s, a);
    return hipGetLastError();
}

}  // namespace cq
