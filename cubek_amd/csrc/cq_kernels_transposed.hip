// Quantize / dequantize when the float tensor is stored transposed: its memory-fastest
// dimension is the second to last logical one (a [.., R, C] view of a [.., C, R]
// buffer), while blocks and packing run along C.  The reference reaches such tensors
// through strided linear views with line size 1 (crates/cubek-quant/src/quantize.rs:309-317).
//
// A wave holds 64 consecutive r of one block (or, per tensor, one 32-column segment): lane
// l walks the block's columns for its own r, so every load or store of floats is one
// contiguous run across the wave, and the abs-max of a block never leaves the thread.
// Column addresses are wave-uniform (scalar registers) plus a 32-bit lane offset.  Blocks of
// up to 32 columns stay in registers between the abs-max and the quantize pass; blocks of 64
// or 128 columns are shared by 2 or 4 lanes (quantize_transposed_quads_kernel); longer ones
// are read twice, the second time from cache.  Stored words are written / read per thread (a
// few words per row and block, rows far apart): that side moves 1/4 - 1/16 of the bytes.
//
// Kernels: quantize_transposed_kernel (given scales or fused abs-max), its variant
// quantize_transposed_quads_kernel, scales_transposed_kernel (abs-max -> scale only),
// dequantize_transposed_kernel.
#include "cq_device.hpp"
#include "cq_internal.hpp"
#include "cq_magic_div.hpp"

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

// A wave's place: 64 consecutive r (one per lane) of segment `seg`.  seg is the same for the whole
// wave, and said so to the compiler, so that everything derived from it stays in scalar registers
// and a float access is "scalar base + 32-bit lane offset" with no address arithmetic per lane.
struct Lane {
    uint32_t r, seg;
    uint32_t byte;  // lane's offset from the wave's first r, in bytes
    bool live;
};
template <class F>
__device__ __forceinline__ Lane lane_of(const TransposedArgs& a) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    Lane t;
    t.r = blockIdx.x * kWave + lane;
    t.seg = __builtin_amdgcn_readfirstlane(blockIdx.y * kSegmentsPerGroup + threadIdx.x / kWave);
    t.byte = lane * F::kBytes;
    t.live = t.r < a.rows && t.seg < a.segments;
    return t;
}
// A wave-uniform address handed over as a scalar value of its own (64-bit products come out of
// the vector unit, and the compiler otherwise folds the lane offset into the base first and
// computes every column's address per lane).  Rebuilt as a pointer into global memory, which it
// is: a bare integer would become a flat pointer.
__device__ __forceinline__ const char* scalar_address(const char* ptr) {
    const uint64_t p = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(p));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(p >> 32));
    typedef const char __attribute__((address_space(1))) * GlobalPtr;
    return (const char*)(GlobalPtr)(static_cast<uint64_t>(hi) << 32 | lo);
}
// address of (first r of the wave, column c0) / of column c0 + c in the same rows
template <class F>
__device__ __forceinline__ const char* wave_base(const void* base, const TransposedArgs& a, uint64_t batch, uint32_t c0) {
    return scalar_address(static_cast<const char*>(base) +
                          (batch + static_cast<uint64_t>(blockIdx.x) * kWave + static_cast<uint64_t>(c0) * a.pitch_f) * F::kBytes);
}
template <class F>
__device__ __forceinline__ const char* column(const char* base, const TransposedArgs& a, uint32_t c) {
    return scalar_address(base + static_cast<uint64_t>(c) * a.pitch_f * F::kBytes);
}

// f32 value -> the bits of an element of F (rounded to nearest even)
template <class F>
__device__ __forceinline__ uint32_t element_bits(float v) {
    if constexpr (F::kBytes == 4) {
        return f32_bits(v);
    } else if constexpr (F::kDtype == CQ_BF16) {
        return BF16::pack2(v, 0.0f) & 0xffffu;
    } else {
        return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, F16::narrow(v)));
    }
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

// kPiece (32 or 16) values of one row -> codes -> the piece's stored words
template <class F, int kBits, bool kWide, int kEnc, uint32_t kPiece = 32>
__device__ __forceinline__ void quantize_piece_words(const float* v, float d, bool tame, const QuantParams& qp, uint32_t* pw) {
    using U = Unit<F, kBits>;
    constexpr int kN = U::kN;
    static_assert(kPiece % U::kV == 0, "a piece is whole units");
#pragma unroll
    for (uint32_t u = 0; u < kPiece / U::kV; u++) {
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < U::kChunks; i++) {
            float qn[kN];
            quantize_codes<F, kN, kEnc>(v + u * U::kV + i * kN, d, tame, qp.lo, qp.hi, qp.unrounded != 0, qn);
            uint32_t cw[2] = {0, 0};
            if constexpr (kEnc == kEncInt)
                pack_chunk_neg<kBits, kN, kWide>(qn, cw);
            else
                encode_chunk<kEnc, kN>(qn, cw);
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
}
// ... and `valid` of them stored at `out`
template <class F, int kBits, bool kWide, int kEnc>
__device__ __forceinline__ void quantize_piece(const float* v, float d, bool tame, const QuantParams& qp, uint32_t* out,
                                               uint32_t valid) {
    constexpr int kPieceWords = 32 / Unit<F, kBits>::kNq;
    uint32_t pw[kPieceWords];
    quantize_piece_words<F, kBits, kWide, kEnc>(v, d, tame, qp, pw);
    store_words<kPieceWords>(out, pw, valid);
}

// kScale: 0 dynamic (abs-max of the block), 1 given (scale_in typed scale_in_dtype)
template <class F, int kBits, bool kWide, int kEnc, int kScale>
__global__ __launch_bounds__(kThreads) void quantize_transposed_kernel(TransposedArgs a, QuantParams qp) {
    using U = Unit<F, kBits>;
    const Lane t = lane_of<F>(a);
    if (!t.live) return;  // nothing below needs the whole wave
    const uint32_t r = t.r, seg = t.seg;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t c0 = seg * a.segment;
    const char* in0 = wave_base<F>(a.input, a, b.f, c0);

    // a piece = up to 32 columns of the segment held in registers (32 loads in flight per lane)
    constexpr uint32_t kPiece = 32;
    static_assert(kPiece % U::kV == 0, "pieces hold whole units");
    float v[kPiece];
    const auto load_piece = [&](uint32_t c) {
        if (c + kPiece <= a.segment) {
#pragma unroll
            for (uint32_t i = 0; i < kPiece; i++) v[i] = F::load(column<F>(in0, a, c + i) + t.byte, 0);
        } else {
#pragma unroll
            for (uint32_t i = 0; i < kPiece; i++) {
                v[i] = 0.0f;
                if (c + i < a.segment) v[i] = F::load(column<F>(in0, a, c + i) + t.byte, 0);
            }
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
        const uint32_t left = a.segment - c;
        quantize_piece<F, kBits, kWide, kEnc>(v, d, tame, qp, out + c / U::kNq, left >= kPiece ? kPiece / U::kNq : left / U::kNq);
    }
}

// Quads of lanes, for 8-byte aligned runs.  Blocks of 64 or 128 columns: the lane-per-row kernel
// above would read them twice (abs-max, then quantize, 32 columns at a time); here 2 or 4
// neighbouring lanes share a block, 32 columns each, and combine their maxima through DPP, so a
// block is read once and stays in registers.  Blocks of 32 columns: four neighbouring lanes hold
// four neighbouring blocks of the same rows, so the words and scales of a row sit side by side.
// The four waves of a workgroup sit side by side along the columns too and hand their words and
// f32 scales over through LDS, from where a tile's rows leave as whole runs (256 bytes of 4-bit
// codes, 64 bytes of scales per row) rather than one request per lane; outputs that are not
// 16-byte aligned are stored by each quad for itself.
// To keep the float runs long with fewer lanes along r, a lane holds kR = 2 (f32) or 4 (16-bit
// types) consecutive r through one 8-byte load: a wave covers 16 * kR rows by 128 columns and a
// load instruction fetches four runs of 128 bytes.  Needs 8-byte aligned runs (base address,
// pitch, batch strides), a row count that is a multiple of kR and 128 columns within 2 GiB of
// each other.
template <class F>
constexpr int kRowsPerLane = 8 / F::kBytes;
constexpr int kQuad = 4;

// element j of the kR a lane loaded together
template <class F>
__device__ __forceinline__ float lane_row(u32x2 raw, int j) {
    if constexpr (F::kBytes == 4) {
        return bits_f32(raw[j]);
    } else {
        const uint32_t w = raw[j >> 1];
        if constexpr (F::kDtype == CQ_BF16) {
            return bits_f32((j & 1) ? (w & 0xffff0000u) : (w << 16));
        } else {
            const f16x2 h = __builtin_bit_cast(f16x2, w);
            return static_cast<float>(h[j & 1]);
        }
    }
}

// Eight words per lane (32 columns of 8-bit codes), four lanes side by side = 128 contiguous
// bytes: written as two instructions of 64 contiguous bytes per quad instead of two of 4 x 16
// scattered ones.  Piece q (16 bytes) of the run sits in lane q / 2, words 4 * (q % 2)...; in
// instruction k lane s writes piece 4 k + s.  `run` is the quad's first word; all four lanes
// of the quad are here.
__device__ __forceinline__ void store_quad_run(uint32_t* run, const uint32_t* pw, uint32_t s) {
    constexpr int kFrom01 = 0x50, kFrom23 = 0xfa;  // quad_perm [0,0,1,1] and [2,2,3,3]
    const bool upper = (s & 1u) != 0;
#pragma unroll
    for (int k = 0; k < 2; k++) {
        u32x4 piece;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t lo = k == 0 ? dpp<kFrom01>(pw[w]) : dpp<kFrom23>(pw[w]);
            const uint32_t hi = k == 0 ? dpp<kFrom01>(pw[4 + w]) : dpp<kFrom23>(pw[4 + w]);
            piece[w] = upper ? hi : lo;
        }
        *reinterpret_cast<u32x4*>(run + (4 * k + s) * 4) = piece;
    }
}

template <class F, int kBits, bool kWide, int kEnc, int kScale>
__global__ __launch_bounds__(kThreads) void quantize_transposed_quads_kernel(TransposedArgs a, QuantParams qp) {
    using U = Unit<F, kBits>;
    constexpr int kR = kRowsPerLane<F>;
    constexpr uint32_t kPart = 32;                 // columns per lane
    constexpr uint32_t kLaneRows = kWave / kQuad;  // lanes along r
    constexpr uint32_t kPartWords = kPart / U::kNq;
    // the workgroup's tile: its four waves sit side by side along the columns
    constexpr uint32_t kTileRows = kLaneRows * kR;
    constexpr uint32_t kTileParts = kQuad * kSegmentsPerGroup;
    constexpr uint32_t kRowWords = kTileParts * kPartWords;
    constexpr uint32_t kRowPitch = kRowWords + 4;  // rows start four banks apart
    __shared__ __attribute__((aligned(16))) uint32_t lds_words[kTileRows * kRowPitch];
    __shared__ uint32_t lds_scales[kTileRows * kTileParts];

    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t s = lane & (kQuad - 1);
    const uint32_t lr = lane / kQuad;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t r0 = (blockIdx.x * kLaneRows + lr) * kR;
    // parts of 32 columns: the tile's first, the quad's first, the lane's own; a block is 1, 2 or 4
    // parts, so the lanes of a block sit in one quad
    const uint32_t tile_part0 = blockIdx.y * kTileParts;
    const uint32_t part0 = tile_part0 + wave * kQuad;
    const uint32_t parts_per_block = a.segment / kPart;
    const uint32_t parts = a.segments * parts_per_block;
    const BatchPos b = batch_pos(a, blockIdx.z);
    if (r0 < a.rows && part0 + s < parts) {  // rows is a multiple of kR: a lane's rows all exist
        const bool whole_quad = part0 + kQuad <= parts;  // else blocks of two parts, and only the first is here
        const uint32_t seg = (part0 + s) / parts_per_block;
        const bool first_part = (s & (parts_per_block - 1)) == 0;
        const char* in0 = scalar_address(static_cast<const char*>(a.input) +
                                         (b.f + static_cast<uint64_t>(blockIdx.x) * kLaneRows * kR +
                                          static_cast<uint64_t>(part0) * kPart * a.pitch_f) * F::kBytes);
        // the lane's own corner: its part's first column, its first r (below 2 GiB, the launcher checks)
        const uint32_t corner = s * kPart * static_cast<uint32_t>(a.pitch_f) * F::kBytes + lr * 8;

        u32x2 raw[kPart];
#pragma unroll
        for (uint32_t i = 0; i < kPart; i++) raw[i] = *reinterpret_cast<const u32x2*>(column<F>(in0, a, i) + corner);

        float d[kR];
#pragma unroll
        for (int j = 0; j < kR; j++) {
            float s_f;
            if constexpr (kScale == 0) {
                float amax = 0.0f;
#pragma unroll
                for (uint32_t i = 0; i < kPart; i++) amax = fmaxf(amax, fabsf(lane_row<F>(raw[i], j)));  // NaN elements drop out
                uint32_t bits = f32_bits(amax);  // non-negative floats order like their bits
                if (parts_per_block >= 2) bits = max(bits, dpp<kDppXor1>(bits));
                if (parts_per_block >= kQuad) bits = max(bits, dpp<kDppXor2>(bits));
                amax = bits_f32(bits);
                const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
                s_f = F::round(s32);
            } else {
                const uint64_t si = a.tensor_level ? 0 : b.sa + static_cast<uint64_t>(r0 + j) * a.sa_row + static_cast<uint64_t>(seg) * a.sa_col;
                s_f = load_dtype(a.scale_in_dtype, a.scale_in, si);
            }
            const float s_fs = round_to_dtype(a.param_dtype, s_f);  // write_scale (src/quantize.rs:83-98)
            if (a.scale_out != nullptr && first_part) {
                if (a.tensor_level) {
                    if (b.first && r0 + j == 0 && part0 + s == 0) store_dtype(a.param_dtype, a.scale_out, 0, s_fs);
                } else if (a.staged & 2u) {
                    lds_scales[(lr * kR + j) * kTileParts + (wave * kQuad + s) / parts_per_block] = f32_bits(s_fs);
                } else {
                    store_dtype(a.param_dtype, a.scale_out,
                                b.sb + static_cast<uint64_t>(r0 + j) * a.sb_row + static_cast<uint64_t>(seg) * a.sb_col, s_fs);
                }
            }
            d[j] = F::round(s_fs);
        }

        uint32_t* run = static_cast<uint32_t*>(a.output) + b.v + static_cast<uint64_t>(r0) * a.vrow + part0 * kPartWords;
#pragma unroll
        for (int j = 0; j < kR; j++) {
            float v[kPart];
#pragma unroll
            for (uint32_t i = 0; i < kPart; i++) v[i] = lane_row<F>(raw[i], j);
            uint32_t pw[kPartWords];
            quantize_piece_words<F, kBits, kWide, kEnc>(v, d[j], divisor_is_tame(d[j]), qp, pw);
            uint32_t* row_run = run + j * a.vrow;
            if (a.staged & 1u)
                store_words<kPartWords>(&lds_words[(lr * kR + j) * kRowPitch + (wave * kQuad + s) * kPartWords], pw, kPartWords);
            else if (kPartWords == 8 && whole_quad && (reinterpret_cast<uintptr_t>(row_run) & 15u) == 0)
                store_quad_run(row_run, pw, s);
            else
                store_words<kPartWords>(row_run + s * kPartWords, pw, kPartWords);
        }
    }
    if (a.staged == 0) return;  // the same for every thread of the launch

    // the tile's words and scales leave as whole rows of the tile: 16-byte pieces side by side
    __syncthreads();
    const uint32_t tile_r0 = blockIdx.x * kTileRows;
    const uint32_t rows_here = a.rows - tile_r0 < kTileRows ? a.rows - tile_r0 : kTileRows;
    if (a.staged & 1u) {
        const uint32_t words_here = (parts - tile_part0) * kPartWords < kRowWords ? (parts - tile_part0) * kPartWords : kRowWords;
        uint32_t* tile_out = static_cast<uint32_t*>(a.output) + b.v + static_cast<uint64_t>(tile_r0) * a.vrow + tile_part0 * kPartWords;
#pragma unroll
        for (uint32_t idx = threadIdx.x; idx < kTileRows * (kRowWords / 4); idx += kThreads) {
            const uint32_t row = idx / (kRowWords / 4), q = idx % (kRowWords / 4);
            if (row < rows_here && q * 4 < words_here)  // the launcher checked: rows hold a multiple of four words
                stream_store(*reinterpret_cast<const u32x4*>(&lds_words[row * kRowPitch + q * 4]),
                             reinterpret_cast<u32x4*>(tile_out + static_cast<uint64_t>(row) * a.vrow + q * 4));
        }
    }
    if (a.staged & 2u) {
        const uint32_t tile_seg0 = tile_part0 / parts_per_block;
        const uint32_t tile_segs = kTileParts / parts_per_block;
        const uint32_t segs_here = a.segments - tile_seg0 < tile_segs ? a.segments - tile_seg0 : tile_segs;
        float* tile_scales = static_cast<float*>(a.scale_out) + b.sb + tile_seg0;  // f32, contiguous along the blocks of a row
#pragma unroll
        for (uint32_t idx = threadIdx.x; idx < kTileRows * kTileParts; idx += kThreads) {
            const uint32_t row = idx / kTileParts, i = idx % kTileParts;
            if (row < rows_here && i < segs_here)
                tile_scales[static_cast<uint64_t>(tile_r0 + row) * a.sb_row + i] = bits_f32(lds_scales[row * kTileParts + i]);
        }
    }
}

// Tiles through LDS, for runs of 16 bytes along r: the float side and the stored side both move whole runs.
// The kernels above keep a block's floats in registers (64 - 128 of them per lane, two waves per SIMD, loads
// and arithmetic of a wave taking turns); here the registers hold only what is in flight.  A workgroup owns
// kTileRows = 128 (16-bit types) or 64 (f32) rows and walks its columns 64 at a time.  Per step: every thread
// loads four 16-byte pieces (a wave: four columns by 256 bytes) into registers, which go to LDS behind a
// barrier while the next step's loads are already on their way; then a thread takes 16 columns of one LDS
// word of rows (two rows of a 16-bit type: 16 conflict-free ds_read_b32), quantizes them as the other kernels
// do, and leaves words and scales in LDS.  After the last step the tile's words leave as runs of 128 bytes
// per row, its scales as runs of up to 32.
template <class F>
constexpr uint32_t kTileRowsPerThread = 4 / F::kBytes;
constexpr uint32_t kTilePart = 32;  // columns of the smallest block the tile kernels take

// Which tile a workgroup of the tile kernels takes.  Workgroup i of a launch runs on XCD i % 8, each with an L2 of
// its own: XCD x takes the x-th eighth of the tiles, in order, rows fastest, so that the 256-byte runs which
// neighbouring row tiles read or write in the same columns pass through one L2 at about the same time.
// The grid is (8 * ceil(tiles / 8), 1, batches); workgroups beyond the last tile leave at once.
struct TilePlace {
    uint32_t row_tile, col_tile;
    bool live;
};
__device__ __forceinline__ TilePlace tile_place(uint32_t row_tiles, uint32_t col_tiles) {
    const uint32_t total = row_tiles * col_tiles, per_xcd = gridDim.x / 8;
    const uint32_t tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    return TilePlace{tile % row_tiles, tile / row_tiles, tile < total};
}

// The quantize tile kernel in steps of 64 columns: thread (row pair, 16 columns), two neighbouring lanes share a
// block of 32 columns (their maxima meet by DPP), 128 bytes of codes per row and tile.  16 KiB of floats, 18 KiB of
// words and 4 KiB of scales per workgroup: four workgroups fit a compute unit instead of two.
constexpr uint32_t kQStepCols = 64, kQPart = 16;
template <class F, int kBits, int kEnc, int kScale>
// seg_magic / seg_shift: column / a.segment as a multiplication and a shift (cq_magic_div.hpp; columns below 2^31)
__global__ __launch_bounds__(kThreads) void quantize_transposed_tile_kernel(TransposedArgs a, QuantParams qp, uint32_t seg_magic,
                                                                            uint32_t seg_shift) {
    using U = Unit<F, kBits>;
    constexpr uint32_t kRp = kTileRowsPerThread<F>;
    constexpr uint32_t kTileRows = 64 * kRp;
    constexpr uint32_t kRowWords = 32;                                // 128 bytes of codes per row and tile
    constexpr uint32_t kTileCols = kRowWords * U::kNq;
    constexpr uint32_t kSteps = kTileCols / kQStepCols;
    constexpr uint32_t kPartWords = kQPart / U::kNq;
    static_assert(kPartWords >= 1, "a thread's sixteen columns are whole words");
    constexpr uint32_t kStepWords = kQStepCols / U::kNq;
    constexpr uint32_t kRowParts = kTileCols / kTilePart;            // blocks of 32 columns per row and tile
    constexpr uint32_t kPieceRows = 16 / F::kBytes;                  // rows of one 16-byte piece
    constexpr uint32_t kRowPitch = kRowWords + 4;                    // rows start four banks apart
    constexpr uint32_t kHeld = kQStepCols * 16 / kThreads;           // 16-byte pieces a thread loads per step
    __shared__ __attribute__((aligned(16))) uint32_t lds_floats[kQStepCols * 64];  // [column][word of rows, rotated]
    __shared__ __attribute__((aligned(16))) uint32_t lds_words[kTileRows * kRowPitch];
    __shared__ uint32_t lds_scales[kTileRows * kRowParts];

    const uint32_t t = threadIdx.x;
    const uint32_t cols = a.segments * a.segment;
    const TilePlace place = tile_place((a.rows + kTileRows - 1) / kTileRows, (cols + kTileCols - 1) / kTileCols);
    if (!place.live) return;  // the whole workgroup
    const uint32_t tile_r0 = place.row_tile * kTileRows;
    const uint32_t tile_c0 = place.col_tile * kTileCols;
    const uint32_t parts_per_block = a.segment / kTilePart;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t steps_left = (cols - tile_c0 + kQStepCols - 1) / kQStepCols;
    const uint32_t total = steps_left < kSteps ? steps_left : kSteps;
    const uint32_t rows_here = a.rows - tile_r0 < kTileRows ? a.rows - tile_r0 : kTileRows;

    // loads: piece `piece` (16 bytes of rows) of column i * 16 + t / 16 of the step.  A step's address is a base
    // that is the same for the whole workgroup plus 32 bits per thread (the launcher checked that 64 columns
    // span less than 4 GiB); threads past the tensor's edge re-read the step's first piece, which nobody stores.
    const uint32_t piece = t & 15u, col_sub = t >> 4;
    const bool rows_live = tile_r0 + piece * kPieceRows < a.rows;    // rows is a multiple of kPieceRows
    const char* const in_tile = static_cast<const char*>(a.input) + (b.f + tile_r0) * F::kBytes;
    const uint64_t col_bytes = a.pitch_f * F::kBytes;
    const uint32_t off0 = col_sub * static_cast<uint32_t>(col_bytes) + piece * 16u;
    u32x4 held[kHeld];
    const auto load_step = [&](uint32_t step) {
        const uint32_t step_c0 = tile_c0 + step * kQStepCols;
        const char* const base = in_tile + step_c0 * col_bytes;
        const uint32_t cols_left = cols - step_c0;
#pragma unroll
        for (uint32_t i = 0; i < kHeld; i++) {
            const bool live = rows_live && i * 16 + col_sub < cols_left;
            const uint32_t off = off0 + i * 16u * static_cast<uint32_t>(col_bytes);
            held[i] = stream_load(reinterpret_cast<const u32x4*>(base + (live ? off : 0u)));
        }
        __builtin_amdgcn_sched_barrier(0);  // the loads go out here, a step ahead of their use
    };
    // arithmetic: rows rp * kRp ..., columns part * 16 ... of the step; lanes 2k and 2k + 1 share a block of 32
    const uint32_t part = t & 3u, rp = t >> 2;
    const uint32_t row0 = tile_r0 + rp * kRp;
    const uint32_t word_of_rows = rp ^ (part << 4);  // this thread's place in every column of its group

    load_step(0);
    for (uint32_t step = 0; step < total; step++) {
        __syncthreads();  // the previous step's readers are done with the floats
#pragma unroll
        for (uint32_t i = 0; i < kHeld; i++)
            *reinterpret_cast<u32x4*>(&lds_floats[(i * 16 + col_sub) * 64 + ((piece * 4) ^ (i << 4))]) = held[i];
        __syncthreads();
        if (step + 1 < total) load_step(step + 1);

        const uint32_t c0 = tile_c0 + step * kQStepCols + part * kQPart;
        const bool live = row0 < a.rows && c0 < cols;  // rows is a multiple of kRp
        uint32_t raw[kQPart];
#pragma unroll
        for (uint32_t i = 0; i < kQPart; i++) raw[i] = lds_floats[(part * kQPart + i) * 64 + word_of_rows];
        // the fused abs-max is launched for blocks of 32 columns only; other block sizes divide by multiplication
        const uint32_t seg = kScale == 0 ? c0 / kTilePart : magic_div(c0, seg_magic, seg_shift);
        const uint32_t segment = kScale == 0 ? kTilePart : a.segment;
        const bool first_part = c0 == seg * segment;
        const uint32_t scale_slot = seg - (kScale == 0 ? tile_c0 / kTilePart : magic_div(tile_c0, seg_magic, seg_shift));
#pragma unroll
        for (uint32_t j = 0; j < kRp; j++) {
            float v[kQPart];
#pragma unroll
            for (uint32_t i = 0; i < kQPart; i++) {
                if constexpr (F::kBytes == 4) {
                    v[i] = bits_f32(raw[i]);
                } else if constexpr (F::kDtype == CQ_BF16) {
                    v[i] = bits_f32(j == 0 ? raw[i] << 16 : raw[i] & 0xffff0000u);
                } else {
                    const f16x2 h = __builtin_bit_cast(f16x2, raw[i]);
                    v[i] = static_cast<float>(h[j]);
                }
            }
            float s_f;
            if constexpr (kScale == 0) {  // blocks of 32 columns: two lanes
                float amax = 0.0f;
#pragma unroll
                for (uint32_t i = 0; i < kQPart; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
                amax = group_max<2>(amax);
                const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
                s_f = F::round(s32);
            } else {
                const uint64_t si = a.tensor_level || !live ? 0 : b.sa + static_cast<uint64_t>(row0 + j) * a.sa_row +
                                                                         static_cast<uint64_t>(seg) * a.sa_col;
                s_f = load_dtype(a.scale_in_dtype, a.scale_in, si);
            }
            const float s_fs = round_to_dtype(a.param_dtype, s_f);  // write_scale (src/quantize.rs:83-98)
            if (a.tensor_level) {
                if (a.scale_out != nullptr && b.first && row0 + j == 0 && c0 == 0) store_dtype(a.param_dtype, a.scale_out, 0, s_fs);
            } else if (first_part) {
                lds_scales[(rp * kRp + j) * kRowParts + scale_slot] = f32_bits(s_fs);
            }
            const float d = F::round(s_fs);
            uint32_t pw[kPartWords];
            quantize_piece_words<F, kBits, false, kEnc, kQPart>(v, d, divisor_is_tame(d), qp, pw);
            store_words<kPartWords>(&lds_words[(rp * kRp + j) * kRowPitch + step * kStepWords + part * kPartWords], pw, kPartWords);
        }
    }
    __syncthreads();
    // the tile's words and scales out of LDS: 8 lanes x 16 bytes per row, then the scales of every row
    const uint32_t words_here = (cols - tile_c0) / U::kNq < kRowWords ? (cols - tile_c0) / U::kNq : kRowWords;
    uint32_t* tile_out = static_cast<uint32_t*>(a.output) + b.v + static_cast<uint64_t>(tile_r0) * a.vrow + tile_c0 / U::kNq;
#pragma unroll
    for (uint32_t idx = t; idx < kTileRows * (kRowWords / 4); idx += kThreads) {
        const uint32_t row = idx / (kRowWords / 4), q = idx % (kRowWords / 4);
        if (row < rows_here && q * 4 < words_here)  // the launcher checked: rows hold a multiple of four words
            stream_store(*reinterpret_cast<const u32x4*>(&lds_words[row * kRowPitch + q * 4]),
                         reinterpret_cast<u32x4*>(tile_out + static_cast<uint64_t>(row) * a.vrow + q * 4));
    }
    if (a.scale_out != nullptr && !a.tensor_level) {
        const uint32_t tile_seg0 = tile_c0 / a.segment;
        const uint32_t tile_segs = kRowParts / parts_per_block;
        const uint32_t segs_here = a.segments - tile_seg0 < tile_segs ? a.segments - tile_seg0 : tile_segs;
#pragma unroll
        for (uint32_t idx = t; idx < kTileRows * kRowParts; idx += kThreads) {
            const uint32_t row = idx / kRowParts, i = idx % kRowParts;
            if (row < rows_here && i < segs_here)
                store_dtype(a.param_dtype, a.scale_out,
                            b.sb + static_cast<uint64_t>(tile_r0 + row) * a.sb_row + static_cast<uint64_t>(tile_seg0 + i) * a.sb_col,
                            bits_f32(lds_scales[row * kRowParts + i]));
        }
    }
}

// Block abs-max -> scale typed `out_dtype` (what cq_compute_scales produces), same mapping.
template <class F>
__global__ __launch_bounds__(kThreads) void scales_transposed_kernel(TransposedArgs a, int out_dtype, QuantParams qp) {
    const Lane t = lane_of<F>(a);
    if (!t.live) return;
    const uint32_t r = t.r, seg = t.seg;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const char* in0 = wave_base<F>(a.input, a, b.f, seg * a.segment);
    constexpr uint32_t kPiece = 32;
    float amax = 0.0f;
    for (uint32_t c = 0; c < a.segment; c += kPiece) {
        float v[kPiece];
        if (c + kPiece <= a.segment) {
#pragma unroll
            for (uint32_t i = 0; i < kPiece; i++) v[i] = F::load(column<F>(in0, a, c + i) + t.byte, 0);
        } else {
#pragma unroll
            for (uint32_t i = 0; i < kPiece; i++) {
                v[i] = 0.0f;
                if (c + i < a.segment) v[i] = F::load(column<F>(in0, a, c + i) + t.byte, 0);
            }
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
    const Lane t = lane_of<F>(a);
    if (!t.live) return;
    const uint32_t r = t.r, seg = t.seg;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t c0 = seg * a.segment;
    char* out0 = const_cast<char*>(wave_base<F>(a.output, a, b.f, c0));
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
                F::store(const_cast<char*>(column<F>(out0, a, c + k * U::kNq + i)) + t.byte, 0, s * y[i]);  // store rounds to F
        }
    }
}

// Dequantize on 8-byte aligned runs.  The 2-byte stores of the lane-per-row kernel reach memory
// through the L2 in no particular order, which holds a tensor that does not sit in the Infinity
// Cache at half the HBM rate; here a lane writes its kR consecutive r of a column as one 8-byte
// non-temporal store (a run of 512 bytes per wave and column) and walks 32 columns.  With 4-bit
// codes, inputs and outputs rotated out of the cache: bf16 [8192, 8192] 32 us against 44 us,
// [28672, 8192] 138 us against 150 us.  Blocks of any multiple of 32 columns, or per tensor.
template <class F, int kBits, int kEnc>
__global__ __launch_bounds__(kThreads) void dequantize_transposed_wide_kernel(TransposedArgs a) {
    using U = Unit<F, kBits>;
    constexpr int kR = kRowsPerLane<F>;
    constexpr uint32_t kPart = 32;
    constexpr uint32_t kPartWords = kPart / U::kNq;
    constexpr int kPerWord = 4 / F::kBytes;  // elements of F per 32-bit word of the 8-byte store
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t r0 = (blockIdx.x * kWave + lane) * kR;
    const uint32_t part = __builtin_amdgcn_readfirstlane(blockIdx.y * kSegmentsPerGroup + threadIdx.x / kWave);  // 32 columns
    const uint32_t parts_per_block = a.segment / kPart;
    if (r0 >= a.rows || part >= a.segments * parts_per_block) return;  // rows is a multiple of kR: a lane's rows all exist
    const uint32_t seg = part / parts_per_block;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const char* out0 = scalar_address(static_cast<const char*>(a.output) +
                                      (b.f + static_cast<uint64_t>(blockIdx.x) * kWave * kR +
                                       static_cast<uint64_t>(part) * kPart * a.pitch_f) * F::kBytes);

    uint32_t w[kR][kPartWords];
    float sc[kR];
    const uint32_t* in = static_cast<const uint32_t*>(a.input) + b.v + static_cast<uint64_t>(r0) * a.vrow + part * kPartWords;
#pragma unroll
    for (int j = 0; j < kR; j++) {
        load_words<kPartWords>(in + j * a.vrow, w[j], kPartWords);
        const uint64_t si = a.tensor_level ? 0 : b.sa + static_cast<uint64_t>(r0 + j) * a.sa_row + static_cast<uint64_t>(seg) * a.sa_col;
        sc[j] = F::round(load_dtype(a.param_dtype, a.scale_in, si));  // Line::cast_from(scale)
    }
    u32x2 raw[kPart];
#pragma unroll
    for (uint32_t i = 0; i < kPart; i++) raw[i] = u32x2{0u, 0u};
#pragma unroll
    for (int j = 0; j < kR; j++) {
#pragma unroll
        for (uint32_t k = 0; k < kPartWords; k++) {
            float y[U::kNq];
            decode_fields<kEnc, kBits, U::kNq>(w[j][k], y);
#pragma unroll
            for (uint32_t i = 0; i < U::kNq; i++)
                raw[k * U::kNq + i][j / kPerWord] |= element_bits<F>(sc[j] * y[i]) << (32 / kPerWord * (j % kPerWord));
        }
    }
#pragma unroll
    for (uint32_t i = 0; i < kPart; i++)
        stream_store(raw[i], reinterpret_cast<u32x2*>(const_cast<char*>(column<F>(out0, a, i)) + lane * 8));
}

// The same tile the other way round: a workgroup takes 256 bytes of codes of each of its 64 * kRp rows into LDS in one
// go (16 lanes x 16 bytes per row), then walks the tile 64 columns at a time: thread (row pair, 16 columns)
// decodes its columns of kRp rows and leaves them in LDS as [column][word of rows], and every column leaves as
// 16-byte pieces, 256 bytes per column and step.  Sixteen columns per thread keep the step's floats at 16 KiB, so
// that three workgroups fit a compute unit; the words of a column are stored rotated by its group of sixteen
// columns, which spreads the four column groups of a wave over the banks.  Blocks of any multiple of 32
// columns, or per tensor.
constexpr uint32_t kDeqStepCols = 64, kDeqPart = 16;
template <class F, int kBits, int kEnc>
__global__ __launch_bounds__(kThreads) void dequantize_transposed_tile_kernel(TransposedArgs a, uint32_t seg_magic,
                                                                              uint32_t seg_shift) {
    using U = Unit<F, kBits>;
    constexpr uint32_t kRp = kTileRowsPerThread<F>;
    constexpr uint32_t kTileRows = 64 * kRp;
    constexpr uint32_t kRowWords = 64;                                // 256 bytes of codes per row and tile
    constexpr uint32_t kTileCols = kRowWords * U::kNq;
    constexpr uint32_t kSteps = kTileCols / kDeqStepCols;             // 8 (4-bit), 4 (8-bit), 16 (2-bit)
    constexpr uint32_t kPartWords = kDeqPart / U::kNq;                // words of a thread per row and step
    static_assert(kPartWords >= 1, "a thread's sixteen columns are whole words");
    constexpr uint32_t kStepWords = kDeqStepCols / U::kNq;
    constexpr uint32_t kPieceRows = 16 / F::kBytes;                  // rows of one 16-byte piece
    constexpr uint32_t kRowPitch = kRowWords + 4;                    // rows start four banks apart
    constexpr uint32_t kHeld = kTileRows * (kRowWords / 4) / kThreads;
    constexpr uint32_t kStorePieces = kDeqStepCols * 16 / kThreads;  // 16-byte pieces a thread stores per step
    __shared__ __attribute__((aligned(16))) uint32_t lds_words[kTileRows * kRowPitch];
    __shared__ __attribute__((aligned(16))) uint32_t lds_floats[kDeqStepCols * 64];  // [column][word of rows, rotated]

    const uint32_t t = threadIdx.x;
    const uint32_t cols = a.segments * a.segment;
    const TilePlace place = tile_place((a.rows + kTileRows - 1) / kTileRows, (cols + kTileCols - 1) / kTileCols);
    if (!place.live) return;  // the whole workgroup
    const uint32_t tile_r0 = place.row_tile * kTileRows;
    const uint32_t tile_c0 = place.col_tile * kTileCols;
    const BatchPos b = batch_pos(a, blockIdx.z);
    const uint32_t steps_left = (cols - tile_c0 + kDeqStepCols - 1) / kDeqStepCols;
    const uint32_t total = steps_left < kSteps ? steps_left : kSteps;
    const uint32_t rows_here = a.rows - tile_r0 < kTileRows ? a.rows - tile_r0 : kTileRows;
    const uint32_t words_here = (cols - tile_c0) / U::kNq < kRowWords ? (cols - tile_c0) / U::kNq : kRowWords;

    // every load of the workgroup's codes goes out first
    const uint32_t* tile_in = static_cast<const uint32_t*>(a.input) + b.v + static_cast<uint64_t>(tile_r0) * a.vrow + tile_c0 / U::kNq;
    u32x4 held[kHeld];
#pragma unroll
    for (uint32_t k = 0; k < kHeld; k++) {
        const uint32_t idx = k * kThreads + t, row = idx / (kRowWords / 4), q = idx % (kRowWords / 4);
        const bool live = row < rows_here && q * 4 < words_here;  // the launcher checked: rows hold a multiple of four words
        held[k] = live ? stream_load(reinterpret_cast<const u32x4*>(tile_in + static_cast<uint64_t>(live ? row : 0) * a.vrow + (live ? q * 4 : 0)))
                       : u32x4{0u, 0u, 0u, 0u};
    }
    // thread (rp, part): rows rp * kRp ..., columns part * 16 ... of every step
    const uint32_t part = t & 3u, rp = t >> 2;
    const uint32_t row0 = tile_r0 + rp * kRp;
    const bool row_live = row0 < a.rows;  // rows is a multiple of kRp
    const char* const scale0 = static_cast<const char*>(a.scale_in);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (uint32_t k = 0; k < kHeld; k++) {
        const uint32_t idx = k * kThreads + t, row = idx / (kRowWords / 4), q = idx % (kRowWords / 4);
        *reinterpret_cast<u32x4*>(&lds_words[row * kRowPitch + q * 4]) = held[k];
    }

    // stores: piece `piece` (16 bytes of rows) of column i * 16 + t / 16 of the step
    const uint32_t piece = t & 15u, col_sub = t >> 4;
    const bool rows_live = tile_r0 + piece * kPieceRows < a.rows;    // rows is a multiple of kPieceRows
    char* const out0 = static_cast<char*>(a.output) + (b.f + tile_r0 + static_cast<uint64_t>(piece) * kPieceRows) * F::kBytes;
    for (uint32_t step = 0; step < total; step++) {
        // the scales of this thread's rows for the step (the words are on their way or there already)
        const uint32_t c0 = tile_c0 + step * kDeqStepCols + part * kDeqPart;
        const bool live = row_live && c0 < cols && !a.tensor_level;
        RawScale raw_scale[kRp];
#pragma unroll
        for (uint32_t j = 0; j < kRp; j++) {
            const uint64_t si = live ? b.sa + static_cast<uint64_t>(row0 + j) * a.sa_row +
                                           static_cast<uint64_t>(magic_div(c0, seg_magic, seg_shift)) * a.sa_col
                                     : 0;
            raw_scale[j] = load_dtype_raw(a.param_dtype, scale0, si);
        }
        __syncthreads();  // the words are in LDS (first step); the previous step's columns have left the floats
        uint32_t w[kRp][kPartWords];
#pragma unroll
        for (uint32_t j = 0; j < kRp; j++)
            load_words<kPartWords>(&lds_words[(rp * kRp + j) * kRowPitch + step * kStepWords + part * kPartWords], w[j], kPartWords);
        float sc[kRp];
#pragma unroll
        for (uint32_t j = 0; j < kRp; j++) sc[j] = F::round(widen_dtype_raw(a.param_dtype, raw_scale[j]));  // Line::cast_from(scale)
        const uint32_t word_of_rows = rp ^ (part << 4);  // this thread's place in every column of its group
#pragma unroll
        for (uint32_t k = 0; k < kPartWords; k++) {
            float y[kRp][U::kNq];
#pragma unroll
            for (uint32_t j = 0; j < kRp; j++) decode_fields<kEnc, kBits, U::kNq>(w[j][k], y[j]);
#pragma unroll
            for (uint32_t i = 0; i < U::kNq; i++) {
                uint32_t word;
                if constexpr (F::kBytes == 4) {
                    word = f32_bits(sc[0] * y[0][i]);
                } else if constexpr (F::kDtype == CQ_BF16) {
                    word = BF16::pack2(sc[0] * y[0][i], sc[kRp - 1] * y[kRp - 1][i]);
                } else {
                    word = element_bits<F>(sc[0] * y[0][i]) | element_bits<F>(sc[kRp - 1] * y[kRp - 1][i]) << 16;
                }
                lds_floats[(part * kDeqPart + k * U::kNq + i) * 64 + word_of_rows] = word;
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t i = 0; i < kStorePieces; i++) {
            const uint32_t lc = i * 16 + col_sub;  // column of the step; its group of sixteen is i
            const uint32_t c = tile_c0 + step * kDeqStepCols + lc;
            if (rows_live && c < cols)
                stream_store(*reinterpret_cast<const u32x4*>(&lds_floats[lc * 64 + ((piece * 4) ^ (i << 4))]),
                             reinterpret_cast<u32x4*>(out0 + static_cast<uint64_t>(c) * a.pitch_f * F::kBytes));
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

// 8-byte runs along r for the kernels that hold kR rows per lane
template <class F>
bool runs_of_8_bytes(const TransposedArgs& a, const void* floats) {
    bool ok = a.rows % kRowsPerLane<F> == 0 && (reinterpret_cast<uintptr_t>(floats) & 7u) == 0 && (a.pitch_f * F::kBytes) % 8 == 0;
    for (uint32_t k = 0; k < a.num_batch_dims; k++) ok = ok && (a.batch_f[k] * F::kBytes) % 8 == 0;
    return ok;
}
// 16-byte runs along r for the kernels that move tiles through LDS
template <class F>
bool runs_of_16_bytes(const TransposedArgs& a, const void* floats) {
    bool ok = a.rows % (16 / F::kBytes) == 0 && (reinterpret_cast<uintptr_t>(floats) & 15u) == 0 && (a.pitch_f * F::kBytes) % 16 == 0;
    for (uint32_t k = 0; k < a.num_batch_dims; k++) ok = ok && (a.batch_f[k] * F::kBytes) % 16 == 0;
    return ok;
}
template <class F, int kScale>
hipError_t quantize_transposed(hipStream_t s, int bits, const TransposedArgs& a) {
    QuantParams qp;
    qp.lo = a.range.lo;
    qp.hi = a.range.hi;
    qp.width = a.range.hi - a.range.lo;
    qp.rwidth = 1.0f / qp.width;  // IEEE division on the host: correctly rounded
    qp.unrounded = a.range.unrounded;
    const bool wide = a.range.hi > 127.0f || a.range.lo < -128.0f;
    // Quads of lanes wherever the runs are 8-byte aligned: blocks of 64 / 128 columns are read once
    // instead of twice, blocks of 32 cost a quarter of the store requests (4-bit codes of a transposed
    // bf16 view [28672, 8192]: 161 us against 214 us; when the tensor sits in the Infinity Cache the
    // lane-per-row kernel is up to 10 % faster, which is given up).  A fused per-tensor launch does
    // not exist: that scale comes from the two-pass reduction.
    constexpr uint32_t kWaveRows = kWave / kQuad * kRowsPerLane<F>;
    const uint32_t parts = a.segments * (a.segment / 32);
    dim3 grid = grid_of(a);
    bool quads = (kScale == 1 || !a.tensor_level) && runs_of_8_bytes<F>(a, a.input) &&
                 (a.segment == 32 || a.segment == 64 || a.segment == 128) &&
                 a.pitch_f * F::kBytes * 128 < (1ull << 31) && (parts + 15) / 16 <= 65535;
    TransposedArgs q = a;
    if (quads) {
        grid = dim3((a.rows + kWaveRows - 1) / kWaveRows, (parts + 15) / 16, a.batches);
        // words and scales through LDS when their runs can be written as 16-byte / 4-byte pieces side by side
        const uint32_t row_words = a.segments * a.segment / (32u / static_cast<uint32_t>(bits));
        bool words = (reinterpret_cast<uintptr_t>(a.output) & 15u) == 0 && a.vrow % 4 == 0 && row_words % 4 == 0;
        for (uint32_t k = 0; k < a.num_batch_dims; k++) words = words && a.batch_v[k] % 4 == 0;
        const bool scales = a.scale_out != nullptr && !a.tensor_level && a.param_dtype == CQ_F32 && a.sb_col == 1;
        q.staged = (words ? 1u : 0u) | (scales ? 2u : 0u);
    }
    // Tiles through LDS wherever the runs are 16-byte aligned on both sides (blocks of 32 columns for the fused
    // abs-max, any multiple of 32 for given scales): 4-bit codes of a transposed bf16 view [28672, 8192],
    // rotated buffers, against the quads kernel.
    const uint32_t cols = a.segments * a.segment;
    uint32_t seg_magic = 0, seg_shift = 0;
    magic_of(a.segment, &seg_magic, &seg_shift);
    const uint32_t tile_cols = 32u * (32u / static_cast<uint32_t>(bits));  // 128 bytes of codes per row
    // A tile stores the scales of the blocks that start in it, as one run per row: blocks divide the tile's columns
    // (a block of 96 columns would straddle two tiles of 256; such layouts take the kernels below).
    bool tiles = cols < (1u << 31) && a.pitch_f * F::kBytes < (1u << 25) && runs_of_16_bytes<F>(a, a.input) && a.segment % kTilePart == 0 && (kScale == 1 || a.segment == kTilePart) &&
                 (a.tensor_level || tile_cols % a.segment == 0) &&
                 (reinterpret_cast<uintptr_t>(a.output) & 15u) == 0 && a.vrow % 4 == 0 &&
                 (cols / (32u / static_cast<uint32_t>(bits))) % 4 == 0 && a.batches <= 65535;
    for (uint32_t k = 0; k < a.num_batch_dims; k++) tiles = tiles && a.batch_v[k] % 4 == 0;
    const uint64_t tile_count = static_cast<uint64_t>((a.rows + 64 * kTileRowsPerThread<F> - 1) / (64 * kTileRowsPerThread<F>)) *
                                ((cols + tile_cols - 1) / tile_cols);
    const dim3 tile_grid(static_cast<uint32_t>((tile_count + 7) / 8 * 8), 1, a.batches);  // see tile_place()
    // two rounds of resident workgroups and more; below that the quads kernel's many small workgroups win
    // (bf16 [4096, 4096], 4-bit: 14.3 us against 16.0 us; [8192, 8192], 2-bit: 43.6 us against 51.1 us)
    if (tile_count >= (1u << 31) || tile_count * a.batches < 1024) tiles = false;
#define CQ_LAUNCH(B, W, E)                                                                                        \
    {                                                                                                             \
        if (tiles && !W)                                                                                          \
            hipLaunchKernelGGL((quantize_transposed_tile_kernel<F, B, E, kScale>), tile_grid, dim3(kThreads), 0, s, a, qp, \
                               seg_magic, seg_shift);                                                             \
        else if (quads)                                                                                           \
            hipLaunchKernelGGL((quantize_transposed_quads_kernel<F, B, W, E, kScale>), grid, dim3(kThreads), 0, s, q, qp); \
        else                                                                                                      \
            hipLaunchKernelGGL((quantize_transposed_kernel<F, B, W, E, kScale>), grid, dim3(kThreads), 0, s, a, qp); \
        return hipGetLastError();                                                                                 \
    }
    switch (a.encoding) {
        case kEncInt:
            if (bits == 2) CQ_LAUNCH(2, false, kEncInt)
            if (bits == 4) CQ_LAUNCH(4, false, kEncInt)
            if (bits == 8 && wide) break;  // ranges wider than their field take the per-element kernels
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
    constexpr uint32_t kWaveRows = kWave * kRowsPerLane<F>;
    const uint64_t parts = static_cast<uint64_t>(a.segments) * (a.segment / 32);
    dim3 grid = grid_of(a);
    const bool wide_rows = a.segment % 32 == 0 && runs_of_8_bytes<F>(a, a.output) &&
                           (parts + kSegmentsPerGroup - 1) / kSegmentsPerGroup <= 65535;
    if (wide_rows)
        grid = dim3((a.rows + kWaveRows - 1) / kWaveRows, static_cast<uint32_t>((parts + kSegmentsPerGroup - 1) / kSegmentsPerGroup),
                    a.batches);
    // Tiles through LDS wherever both sides allow 16-byte accesses
    const uint32_t cols = a.segments * a.segment;
    uint32_t seg_magic = 0, seg_shift = 0;
    magic_of(a.segment, &seg_magic, &seg_shift);
    bool tiles = cols < (1u << 31) && a.segment % kTilePart == 0 && runs_of_16_bytes<F>(a, a.output) && (reinterpret_cast<uintptr_t>(a.input) & 15u) == 0 &&
                 a.vrow % 4 == 0 && (cols / (32u / static_cast<uint32_t>(bits))) % 4 == 0 && a.batches <= 65535;
    for (uint32_t k = 0; k < a.num_batch_dims; k++) tiles = tiles && a.batch_v[k] % 4 == 0;
    const uint32_t tile_cols = 64u * (32u / static_cast<uint32_t>(bits));  // 256 bytes of codes per row
    const uint64_t tile_count = static_cast<uint64_t>((a.rows + 64 * kTileRowsPerThread<F> - 1) / (64 * kTileRowsPerThread<F>)) *
                                ((cols + tile_cols - 1) / tile_cols);
    const dim3 tile_grid(static_cast<uint32_t>((tile_count + 7) / 8 * 8), 1, a.batches);  // see tile_place()
    // 16-bit floats in four rounds of resident workgroups and more: bf16 [28672, 8192], 4-bit, 125 us against 134 us,
    // [8192, 28672] 115 us against 134 us; [8192, 8192] 37 us against 31 us and f32 [8192, 8192] 61 us against 47 us
    // stay with the lane-per-row kernel
    if (F::kBytes != 2 || tile_count >= (1u << 31) || tile_count * a.batches < 2048) tiles = false;
#define CQ_LAUNCH(B, E)                                                                                       \
    {                                                                                                         \
        if constexpr (F::kBytes == 2) {                                                                       \
            if (tiles) {                                                                                      \
                hipLaunchKernelGGL((dequantize_transposed_tile_kernel<F, B, E>), tile_grid, dim3(kThreads), 0, s, a, \
                                   seg_magic, seg_shift);                                                     \
                return hipGetLastError();                                                                     \
            }                                                                                                 \
        }                                                                                                     \
        if (wide_rows)                                                                                   \
            hipLaunchKernelGGL((dequantize_transposed_wide_kernel<F, B, E>), grid, dim3(kThreads), 0, s, a);  \
        else                                                                                                  \
            hipLaunchKernelGGL((dequantize_transposed_kernel<F, B, E>), grid, dim3(kThreads), 0, s, a);       \
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
