// Quantize / dequantize when the float tensor is stored transposed: its memory-fastest
// dimension is the second to last logical one (a [.., R, C] view of a [.., C, R]
// buffer), while blocks and packing run along C.  The reference reaches such tensors
// through strided linear views with line size 1 (crates/cubek-quant/src/quantize.rs:309-317).
//
// A wave holds 64 consecutive r of one block (or, per tensor, one 32-column segment): lane
// l walks the block's columns for its own r, so every load or store of floats is one
// contiguous run across the wave, and the abs-max of a block never leaves the thread.
// A fused dynamic launch reads the block twice (abs-max, then quantize); the second read
// finds the lines in cache.  Stored words are written / read per thread (a few words per
// row and block, rows far apart): that side moves 1/4 - 1/16 of the bytes.
#include "cq_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;
constexpr int kSegmentsPerGroup = kThreads / kWave;

template <class F, int kBits>
struct Unit {
    static constexpr int kN = F::kPerChunk;
    static constexpr int kNq = 32 / kBits;
    static constexpr int kV = kNq > kN ? kNq : kN;
    static constexpr int kChunks = kV / kN;
    static constexpr int kWords = kV / kNq;
};

// offsets of the workgroup's batch entry (leading dimensions), uniform over the workgroup
struct BatchPos {
    uint64_t f, v, sa, sb;
    bool first;
};
__device__ __forceinline__ BatchPos batch_pos(const TransposedArgs& a, uint32_t batch) {
    BatchPos p{0, 0, 0, 0, batch == 0};
    uint32_t rem = batch;
    for (int d = static_cast<int>(a.num_batch_dims) - 1; d >= 0; d--) {
        const uint32_t c = rem % a.batch_shape[d];
        rem /= a.batch_shape[d];
        p.f += static_cast<uint64_t>(c) * a.batch_f[d];
        p.v += static_cast<uint64_t>(c) * a.batch_v[d];
        p.sa += static_cast<uint64_t>(c) * a.batch_sa[d];
        p.sb += static_cast<uint64_t>(c) * a.batch_sb[d];
    }
    return p;
}

// kCount consecutive words of one thread, as one 16- or 8-byte access when the address allows:
// threads of a wave sit in different rows, so every access is a transaction of its own.
template <int kCount>
__device__ __forceinline__ void store_words(uint32_t* dst, const uint32_t* w, uint32_t valid) {
    if constexpr (kCount % 4 == 0) {
        if (valid == kCount && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
#pragma unroll
            for (int k = 0; k < kCount; k += 4)
                *reinterpret_cast<u32x4*>(dst + k) = u32x4{w[k], w[k + 1], w[k + 2], w[k + 3]};
            return;
        }
    } else if constexpr (kCount % 2 == 0) {
        if (valid == kCount && (reinterpret_cast<uintptr_t>(dst) & 7u) == 0) {
#pragma unroll
            for (int k = 0; k < kCount; k += 2) *reinterpret_cast<u32x2*>(dst + k) = u32x2{w[k], w[k + 1]};
            return;
        }
    }
#pragma unroll
    for (int k = 0; k < kCount; k++)
        if (static_cast<uint32_t>(k) < valid) dst[k] = w[k];
}
template <int kCount>
__device__ __forceinline__ void load_words(const uint32_t* src, uint32_t* w, uint32_t valid) {
    if constexpr (kCount % 4 == 0) {
        if (valid == kCount && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
#pragma unroll
            for (int k = 0; k < kCount; k += 4) {
                const u32x4 q = *reinterpret_cast<const u32x4*>(src + k);
                w[k] = q[0], w[k + 1] = q[1], w[k + 2] = q[2], w[k + 3] = q[3];
            }
            return;
        }
    } else if constexpr (kCount % 2 == 0) {
        if (valid == kCount && (reinterpret_cast<uintptr_t>(src) & 7u) == 0) {
#pragma unroll
            for (int k = 0; k < kCount; k += 2) {
                const u32x2 q = *reinterpret_cast<const u32x2*>(src + k);
                w[k] = q[0], w[k + 1] = q[1];
            }
            return;
        }
    }
#pragma unroll
    for (int k = 0; k < kCount; k++) w[k] = static_cast<uint32_t>(k) < valid ? src[k] : 0u;
}

// kScale: 0 dynamic (abs-max of the block), 1 given (scale_in typed scale_in_dtype)
template <class F, int kBits, bool kWide, int kEnc, int kScale>
__global__ __launch_bounds__(kThreads) void quantize_transposed_kernel(TransposedArgs a, QuantParams qp) {
    using U = Unit<F, kBits>;
    constexpr int kN = U::kN;
    const uint32_t r = blockIdx.x * kWave + (threadIdx.x & (kWave - 1));
    const uint32_t seg = blockIdx.y * kSegmentsPerGroup + threadIdx.x / kWave;
    if (r >= a.rows || seg >= a.segments) return;  // nothing below needs the whole wave
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t c0 = seg * a.segment;
    const uint64_t f0 = b.f + r + static_cast<uint64_t>(c0) * a.pitch_f;

    // a piece = up to 32 columns of the segment held in registers (32 loads in flight per lane)
    constexpr uint32_t kPiece = 32;
    static_assert(kPiece % U::kV == 0, "pieces hold whole units");
    float v[kPiece];
    const auto load_piece = [&](uint32_t c) {
#pragma unroll
        for (uint32_t i = 0; i < kPiece; i++) {
            v[i] = 0.0f;
            if (c + i < a.segment) v[i] = F::load(a.input, f0 + static_cast<uint64_t>(c + i) * a.pitch_f);
        }
    };
    const bool single_piece = a.segment <= kPiece;  // then the abs-max pass and the quantize pass share the registers

    float s_f;
    if constexpr (kScale == 0) {
        float amax = 0.0f;
        for (uint32_t c = 0; c < a.segment; c += kPiece) {
            load_piece(c);
#pragma unroll
            for (uint32_t i = 0; i < kPiece; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
        }
        const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
        s_f = F::round(s32);
    } else {
        const uint64_t si = a.tensor_level ? 0 : b.sa + static_cast<uint64_t>(r) * a.sa_row + static_cast<uint64_t>(seg) * a.sa_col;
        s_f = load_dtype(a.scale_in_dtype, a.scale_in, si);
    }
    // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first element
    const float s_fs = round_to_dtype(a.param_dtype, s_f);
    if (a.scale_out != nullptr) {
        if (a.tensor_level) {
            if (b.first && r == 0 && seg == 0) store_dtype(a.param_dtype, a.scale_out, 0, s_fs);
        } else {
            store_dtype(a.param_dtype, a.scale_out,
                        b.sb + static_cast<uint64_t>(r) * a.sb_row + static_cast<uint64_t>(seg) * a.sb_col, s_fs);
        }
    }
    const float d = F::round(s_fs);
    const bool tame = divisor_is_tame(d);

    uint32_t* out = static_cast<uint32_t*>(a.output) + b.v + static_cast<uint64_t>(r) * a.vrow + c0 / U::kNq;
    for (uint32_t c = 0; c < a.segment; c += kPiece) {
        if (kScale != 0 || !single_piece) load_piece(c);  // a second read finds the lines in cache
        constexpr int kPieceWords = kPiece / U::kNq;
        uint32_t pw[kPieceWords];
#pragma unroll
        for (uint32_t u = 0; u < kPiece / U::kV; u++) {
            uint32_t w[2] = {0, 0};
#pragma unroll
            for (int i = 0; i < U::kChunks; i++) {
                float qn[kN];
                quantize_values_neg<F, kN>(v + u * U::kV + i * kN, d, tame, qp.lo, qp.hi, qn);
                uint32_t cw[2] = {0, 0};
                if constexpr (kEnc == kEncInt)
                    pack_chunk_neg<kBits, kN, kWide>(qn, cw);
                else
                    encode_chunk_neg<kEnc, kN>(qn, cw);
                if constexpr (U::kChunks == 1) {
                    w[0] = cw[0];
                    w[1] = cw[1];
                } else {
                    w[0] |= cw[0] << (i * kN * kBits);  // sub-word chunks, upper bits are zero
                }
            }
            pw[u * U::kWords] = w[0];
            if constexpr (U::kWords == 2) pw[u * U::kWords + 1] = w[1];
        }
        const uint32_t left = a.segment - c;
        store_words<kPieceWords>(out + c / U::kNq, pw, left >= kPiece ? kPieceWords : left / U::kNq);
    }
}

// Block abs-max -> scale typed `out_dtype` (what cq_compute_scales produces), same mapping.
template <class F>
__global__ __launch_bounds__(kThreads) void scales_transposed_kernel(TransposedArgs a, int out_dtype, QuantParams qp) {
    const uint32_t r = blockIdx.x * kWave + (threadIdx.x & (kWave - 1));
    const uint32_t seg = blockIdx.y * kSegmentsPerGroup + threadIdx.x / kWave;
    if (r >= a.rows || seg >= a.segments) return;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint64_t f0 = b.f + r + static_cast<uint64_t>(seg) * a.segment * a.pitch_f;
    constexpr uint32_t kPiece = 32;
    float amax = 0.0f;
    for (uint32_t c = 0; c < a.segment; c += kPiece) {
        float v[kPiece];
#pragma unroll
        for (uint32_t i = 0; i < kPiece; i++) {
            v[i] = 0.0f;
            if (c + i < a.segment) v[i] = F::load(a.input, f0 + static_cast<uint64_t>(c + i) * a.pitch_f);
        }
#pragma unroll
        for (uint32_t i = 0; i < kPiece; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
    }
    const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
    store_dtype(out_dtype, a.scale_out, b.sb + static_cast<uint64_t>(r) * a.sb_row + static_cast<uint64_t>(seg) * a.sb_col,
                round_to_dtype(out_dtype, F::round(s32)));
}

template <class F, int kBits, int kEnc>
__global__ __launch_bounds__(kThreads) void dequantize_transposed_kernel(TransposedArgs a) {
    using U = Unit<F, kBits>;
    const uint32_t r = blockIdx.x * kWave + (threadIdx.x & (kWave - 1));
    const uint32_t seg = blockIdx.y * kSegmentsPerGroup + threadIdx.x / kWave;
    if (r >= a.rows || seg >= a.segments) return;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t c0 = seg * a.segment;
    const uint64_t f0 = b.f + r + static_cast<uint64_t>(c0) * a.pitch_f;
    const uint64_t si = a.tensor_level ? 0 : b.sa + static_cast<uint64_t>(r) * a.sa_row + static_cast<uint64_t>(seg) * a.sa_col;
    const float s = F::round(load_dtype(a.param_dtype, a.scale_in, si));  // Line::cast_from(scale)
    const uint32_t* in = static_cast<const uint32_t*>(a.input) + b.v + static_cast<uint64_t>(r) * a.vrow + c0 / U::kNq;
    // all words of up to 32 columns first (their loads in flight together), then the stores
    constexpr uint32_t kPiece = 32;
    constexpr uint32_t kPieceWords = kPiece / U::kNq;
    for (uint32_t c = 0; c < a.segment; c += kPiece) {
        uint32_t w[kPieceWords];
        const uint32_t left = a.segment - c;
        load_words<kPieceWords>(in + c / U::kNq, w, left >= kPiece ? kPieceWords : left / U::kNq);
#pragma unroll
        for (uint32_t k = 0; k < kPieceWords; k++) {
            if (c + k * U::kNq >= a.segment) break;
            float y[U::kNq];
            decode_fields<kEnc, kBits, U::kNq>(w[k], y);
#pragma unroll
            for (uint32_t i = 0; i < U::kNq; i++)
                F::store(a.output, f0 + static_cast<uint64_t>(c + k * U::kNq + i) * a.pitch_f, s * y[i]);  // store rounds to F
        }
    }
}

#define CQ_SWITCH_DTYPE(D, ...)                              \
    switch (D) {                                             \
        case CQ_F32: { using kF = F32; __VA_ARGS__; }        \
        case CQ_BF16: { using kF = BF16; __VA_ARGS__; }      \
        case CQ_F16: { using kF = F16; __VA_ARGS__; }        \
        default: return hipErrorInvalidValue;                \
    }

inline dim3 grid_of(const TransposedArgs& a) {
    return dim3((a.rows + kWave - 1) / kWave, (a.segments + kSegmentsPerGroup - 1) / kSegmentsPerGroup, a.batches);
}

template <class F, int kScale>
hipError_t quantize_transposed(hipStream_t s, int bits, const TransposedArgs& a) {
    QuantParams qp;
    qp.lo = a.range.lo;
    qp.hi = a.range.hi;
    qp.width = a.range.hi - a.range.lo;
    qp.rwidth = 1.0f / qp.width;  // IEEE division on the host: correctly rounded
    const bool wide = a.range.hi > 127.0f || a.range.lo < -128.0f;
#define CQ_LAUNCH(B, W, E)                                                                                       \
    {                                                                                                            \
        hipLaunchKernelGGL((quantize_transposed_kernel<F, B, W, E, kScale>), grid_of(a), dim3(kThreads), 0, s, a, qp); \
        return hipGetLastError();                                                                                \
    }
    switch (a.encoding) {
        case kEncInt:
            if (bits == 2) CQ_LAUNCH(2, false, kEncInt)
            if (bits == 4) CQ_LAUNCH(4, false, kEncInt)
            if (bits == 8 && wide) CQ_LAUNCH(8, true, kEncInt)
            if (bits == 8) CQ_LAUNCH(8, false, kEncInt)
            break;
        case kEncE4M3: if (bits == 8) CQ_LAUNCH(8, false, kEncE4M3) break;
        case kEncE5M2: if (bits == 8) CQ_LAUNCH(8, false, kEncE5M2) break;
        case kEncE2M1: if (bits == 4) CQ_LAUNCH(4, false, kEncE2M1) break;
    }
#undef CQ_LAUNCH
    return hipErrorInvalidValue;
}

template <class F>
hipError_t dequantize_transposed(hipStream_t s, int bits, const TransposedArgs& a) {
#define CQ_LAUNCH(B, E)                                                                                       \
    {                                                                                                         \
        hipLaunchKernelGGL((dequantize_transposed_kernel<F, B, E>), grid_of(a), dim3(kThreads), 0, s, a);     \
        return hipGetLastError();                                                                             \
    }
    switch (a.encoding) {
        case kEncInt:
            if (bits == 2) CQ_LAUNCH(2, kEncInt)
            if (bits == 4) CQ_LAUNCH(4, kEncInt)
            if (bits == 8) CQ_LAUNCH(8, kEncInt)
            break;
        case kEncE4M3: if (bits == 8) CQ_LAUNCH(8, kEncE4M3) break;
        case kEncE5M2: if (bits == 8) CQ_LAUNCH(8, kEncE5M2) break;
        case kEncE2M1: if (bits == 4) CQ_LAUNCH(4, kEncE2M1) break;
    }
#undef CQ_LAUNCH
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_quantize_transposed(hipStream_t s, int dtype, int bits, bool dynamic, const TransposedArgs& a) {
    if (a.rows == 0 || a.segments == 0 || a.batches == 0) return hipSuccess;
    if (dynamic) {
        CQ_SWITCH_DTYPE(dtype, return (quantize_transposed<kF, 0>(s, bits, a)))
    }
    CQ_SWITCH_DTYPE(dtype, return (quantize_transposed<kF, 1>(s, bits, a)))
}

hipError_t launch_scales_transposed(hipStream_t s, int dtype, int out_dtype, const TransposedArgs& a) {
    if (a.rows == 0 || a.segments == 0 || a.batches == 0) return hipSuccess;
    QuantParams qp;
    qp.lo = a.range.lo;
    qp.hi = a.range.hi;
    qp.width = a.range.hi - a.range.lo;
    qp.rwidth = 1.0f / qp.width;  // IEEE division on the host: correctly rounded
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((scales_transposed_kernel<kF>), grid_of(a), dim3(kThreads), 0, s, a,
                                              out_dtype, qp);
                    return hipGetLastError())
}

hipError_t launch_dequantize_transposed(hipStream_t s, int dtype, int bits, const TransposedArgs& a) {
    if (a.rows == 0 || a.segments == 0 || a.batches == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, return dequantize_transposed<kF>(s, bits, a))
}

}  // namespace cq
