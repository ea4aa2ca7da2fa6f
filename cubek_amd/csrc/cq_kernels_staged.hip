// Streaming quantize / dequantize kernels for two kinds of layouts that the flat kernels (cq_kernels_flat.hpp)
// cannot take as they are, at the price of one trip through LDS:
//
//   pieces       blocks whose extent is not a power-of-two number of 16-byte chunks (24, 40, 48 ... values of a
//                16-bit type): a lane holds `per` consecutive chunks of its block, so the abs-max needs no exchange
//                between lanes beyond a power-of-two butterfly.  Loads stay whole 1 KiB runs per wave: they go
//                straight into LDS (global_load_lds_dwordx4), from where every lane picks up its own chunks.
//   scale tiles  scale tensors with any two strides (stored column by column, say): a workgroup takes a tile of
//                16 rows x 64 chunks and moves the tile's scales through LDS, so that the accesses to the scale
//                tensor run along the dimension that is contiguous there.
//
// Same arithmetic as the flat kernels (cq_device.hpp), same results bit for bit.  The reference addresses scales
// through strides and accepts every block that is a multiple of the values per word
// (crates/cubek-quant/src/lib.rs:20-33, src/layout/scales.rs:144-160,234,260-266).
#include "cq_device.hpp"
#include "cq_internal.hpp"
#include "cq_magic_div.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

// LDS images are written and read back through different types
typedef uint32_t u32a __attribute__((may_alias));
typedef uint16_t u16a __attribute__((may_alias));
typedef uint8_t u8a __attribute__((may_alias));
typedef uint32_t u32x2a __attribute__((ext_vector_type(2), may_alias));
typedef uint32_t u32x4a __attribute__((ext_vector_type(4), may_alias));

QuantParams quant_params(const Range& r) {
    QuantParams p;
    p.lo = r.lo;
    p.hi = r.hi;
    p.width = r.hi - r.lo;
    p.rwidth = 1.0f / p.width;  // IEEE division on the host: correctly rounded
    p.unrounded = r.unrounded;
    return p;
}

// The stored bits of one chunk: w[0] (and w[1] for 64 bits of codes), low bits first, as the flat kernels pack them.
template <class F, int kBits, int kEnc>
__device__ __forceinline__ void quantize_chunk(const float* v, float d, bool tame, const QuantParams& qp, uint32_t* w) {
    constexpr int kN = F::kPerChunk;
    w[0] = w[1] = 0;
    if constexpr (F::kDtype == CQ_F16 && kEnc == kEncInt) {
        if (tame) {
            quantize_pack_f16_tame<kBits>(v, d, qp.lo, qp.hi, w);
            return;
        }
    }
    float qn[kN];
    quantize_codes<F, kN, kEnc>(v, d, tame, qp.lo, qp.hi, qp.unrounded != 0, qn);
    if constexpr (kEnc == kEncInt)
        pack_chunk_neg<kBits, kN, false>(qn, w);
    else
        encode_chunk<kEnc, kN>(qn, w);
}

// scale of a block from its abs-max, as F: F(2 * absmax / (hi - lo))  (crates/cubek-quant/tests/suite/symmetric.rs:163-179)
template <class F>
__device__ __forceinline__ float block_scale(float amax, const QuantParams& qp) {
    return F::round(absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width));
}

// ---- pieces ----------------------------------------------------------------------------------------------------
// A wave owns 64 * per consecutive chunks: load u of the wave brings chunks [u * 64, u * 64 + 64) of them into the
// wave's LDS image, 16 bytes per lane and 1 KiB per instruction, without passing through registers; lane l then
// reads chunks l * per ... l * per + per - 1 (per is odd, so the 16-byte reads of a group of 16 lanes fall on
// different banks).  The codes go into a second image, each chunk's at its place in the run, and leave it as whole
// words, consecutive lanes storing consecutive words.  Nothing crosses a wave: no barrier.
template <class F, int kBits, int kEnc, bool kDynamic>
__global__ __launch_bounds__(kThreads) void quantize_pieces_kernel(const u32x4* __restrict__ in, uint32_t* __restrict__ out,
                                                                   const void* __restrict__ scale_in, void* __restrict__ scale_out,
                                                                   uint64_t num_chunks, uint32_t per, uint32_t group_log2,
                                                                   int param_dtype, uint32_t wide_stores, QuantParams qp) {
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;  // 64, 32, 16 or 8
    constexpr int kChunkBytes = kChunkBits / 8;
    extern __shared__ u32x4 lds[];
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), waves = blockDim.x / kWave;
    const uint64_t wave_index = static_cast<uint64_t>(blockIdx.x) * waves + wave;
    const uint32_t wave_chunks = kWave * per;
    const uint64_t chunk0 = wave_index * wave_chunks;
    if (chunk0 >= num_chunks) return;  // the whole wave
    const uint32_t chunks_here = num_chunks - chunk0 < wave_chunks ? static_cast<uint32_t>(num_chunks - chunk0) : wave_chunks;
    u32x4* const in_image = lds + wave * wave_chunks;
    unsigned char* const out_image = reinterpret_cast<unsigned char*>(lds + waves * wave_chunks) + wave * wave_chunks * kChunkBytes;

    for (uint32_t u = 0; u < per; u++) {
        const uint32_t idx = u * kWave + lane;
        const uint32_t c = idx < chunks_here ? idx : chunks_here - 1;  // lanes past the end re-read the last chunk
        __builtin_amdgcn_global_load_lds(in + chunk0 + c, (__attribute__((address_space(3))) void*)(in_image + u * kWave),
                                         16, 0, 2 /* nt */);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    const u32x4a* const mine = reinterpret_cast<const u32x4a*>(in_image) + lane * per;
    const bool live = lane * per < chunks_here;  // pieces are whole: all of its chunks or none
    const uint64_t block = (wave_index * kWave + lane) >> group_log2;
    float s_f;
    if constexpr (kDynamic) {
        float amax = 0.0f;
        for (uint32_t i = 0; i < per; i++) {
            float v[kN];
            F::unpack(mine[i], v);
#pragma unroll
            for (int k = 0; k < kN; k++) amax = fmaxf(amax, fabsf(v[k]));  // NaN elements drop out
        }
        amax = group_max_rt(amax, group_log2);
        s_f = block_scale<F>(amax, qp);
    } else {
        s_f = F::load(scale_in, live ? block : 0);
    }
    // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first lane; the divisor is F(FS(scale))
    const float s_fs = round_to_dtype(param_dtype, s_f);
    if (scale_out != nullptr && live && (lane & ((1u << group_log2) - 1u)) == 0) store_dtype(param_dtype, scale_out, block, s_fs);
    const float d = F::round(s_fs);
    const bool tame = divisor_is_tame(d);
    for (uint32_t i = 0; i < per; i++) {
        float v[kN];
        F::unpack(mine[i], v);
        uint32_t w[2];
        quantize_chunk<F, kBits, kEnc>(v, d, tame, qp, w);
        unsigned char* const at = out_image + (lane * per + i) * kChunkBytes;
        if constexpr (kChunkBits == 64)
            *reinterpret_cast<u32x2a*>(at) = u32x2{w[0], w[1]};
        else if constexpr (kChunkBits == 32)
            *reinterpret_cast<u32a*>(at) = w[0];
        else if constexpr (kChunkBits == 16)
            *reinterpret_cast<u16a*>(at) = static_cast<uint16_t>(w[0]);
        else
            *reinterpret_cast<u8a*>(at) = static_cast<uint8_t>(w[0]);
    }
    // the image is whole words (blocks are: src/lib.rs:20-33); the lanes of a wave run in step, and LDS takes its
    // accesses in order, so every code is in place when the words are read
    const uint32_t words = chunks_here * kChunkBits / 32;
    uint32_t* const dst = out + chunk0 * kChunkBits / 32;
    uint32_t done = 0;
    if (wide_stores) {  // the run starts on a 16-byte boundary (a wave's share is a multiple of 64 bytes)
        const uint32_t quads = words / 4;
        for (uint32_t j = lane; j < quads; j += kWave)
            stream_store(static_cast<u32x4>(reinterpret_cast<const u32x4a*>(out_image)[j]), reinterpret_cast<u32x4*>(dst) + j);
        done = quads * 4;
    }
    for (uint32_t j = done + lane; j < words; j += kWave) stream_store(static_cast<uint32_t>(reinterpret_cast<const u32a*>(out_image)[j]), dst + j);
}

// ---- scale tiles -----------------------------------------------------------------------------------------------
// A tile is kTileRows rows x kColWaves * 64 chunks.  The four waves of a workgroup stand kColWaves side by side along
// the row and 4 / kColWaves on top of each other; a step of the workgroup is that many rows, a lane's chunk the same in
// every step.  kUnroll steps are in flight at a time.
template <int kRows, int kColWaves_, int kUnroll_>
struct TileShape {
    static constexpr int kTileRows = kRows, kColWaves = kColWaves_, kUnroll = kUnroll_;
    static constexpr int kRowWaves = kWaves / kColWaves;
    static constexpr int kTileChunks = kWave * kColWaves;
    static constexpr int kTileChunksLog2 = kColWaves == 1 ? 6 : (kColWaves == 2 ? 7 : 8);
    static constexpr int kSteps = kTileRows / kRowWaves;
    static constexpr int kIters = kSteps / kUnroll;
    static_assert(kSteps % kUnroll == 0 && kIters >= 1, "whole iterations");
};

// Tile row and block column of entry `idx` of a tile's scales, numbered along the dimension that is closer in
// memory in the scale tensor (rows fastest for a tensor stored column by column).
struct TileScale {
    uint32_t row, bc;
};
template <int kTileRows>
__device__ __forceinline__ TileScale tile_scale(uint32_t idx, bool rows_fastest, uint32_t bcols_log2) {
    if (rows_fastest) return TileScale{idx & (kTileRows - 1), idx / kTileRows};
    return TileScale{idx >> bcols_log2, idx & ((1u << bcols_log2) - 1u)};
}

struct TilePlace {
    uint32_t r0, c0;
};
template <class Shape>
__device__ __forceinline__ TilePlace tile_place(uint32_t col_tiles, uint32_t ct_magic, uint32_t ct_shift) {
    const uint32_t row_tile = magic_div(blockIdx.x, ct_magic, ct_shift);
    return TilePlace{row_tile * Shape::kTileRows, (blockIdx.x - row_tile * col_tiles) * Shape::kTileChunks};
}

// Word `idx` of a tile's codes, numbered along the dimension that is closer in memory in the stored tensor.
struct TileWord {
    uint32_t row, wc;
};
template <int kTileRows, int kTileWords>
__device__ __forceinline__ TileWord tile_word(uint32_t idx, bool rows_fastest) {
    if (rows_fastest) return TileWord{idx % kTileRows, idx / kTileRows};
    return TileWord{idx / kTileWords, idx % kTileWords};
}

// LDS: one float per block of the tile, rows one entry further apart than they are long.
// kStageCodes: the stored tensor's last dimension is not the contiguous one (words of the U32 store `stored_col`
// apart): the tile's words pass through a second LDS image and leave along the dimension that is closer in memory.
template <class F, int kBits, int kEnc, bool kDynamic, class Shape, bool kStageCodes>
__global__ __launch_bounds__(kThreads) void quantize_scale_tiles_kernel(ScaleTileArgs a, QuantParams qp, uint32_t col_tiles,
                                                                       uint32_t ct_magic, uint32_t ct_shift) {
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    constexpr int kUnroll = Shape::kUnroll, kIters = Shape::kIters, kTileRows = Shape::kTileRows;
    constexpr int kTileWords = Shape::kTileChunks * kChunkBits / 32, kWordPitch = kTileWords + 1;
    extern __shared__ float lds_scale[];  // given: the divisors F(FS(scale)); else the scales FS(F(scale)) on their way out
    const uint32_t t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
    const uint32_t wave_row = wave / Shape::kColWaves, tile_chunk = (wave % Shape::kColWaves) * kWave + lane;
    const TilePlace place = tile_place<Shape>(col_tiles, ct_magic, ct_shift);
    const uint32_t bcols_log2 = Shape::kTileChunksLog2 - a.group_log2, bcols = 1u << bcols_log2, pitch = bcols + 1;
    const uint32_t bc0 = place.c0 >> a.group_log2, row_blocks = a.row_chunks >> a.group_log2;
    const uint32_t c = place.c0 + tile_chunk;
    const bool col_live = c < a.row_chunks;
    const uint32_t cl = col_live ? c : a.row_chunks - 1;  // lanes past the end re-read the row's last chunk
    const char* const in = static_cast<const char*>(a.input);
    char* const out = static_cast<char*>(a.output);
    [[maybe_unused]] uint32_t* const lds_words = reinterpret_cast<uint32_t*>(lds_scale + kTileRows * pitch);

    // the loads of iteration it + 1 go out before the arithmetic of iteration it
    u32x4 raw[2][kUnroll];
    const auto load = [&](int it) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t row = place.r0 + (it * kUnroll + u) * Shape::kRowWaves + wave_row;
            const uint32_t rl = row < a.rows ? row : a.rows - 1;
            raw[it & 1][u] = stream_load(reinterpret_cast<const u32x4*>(in + static_cast<uint64_t>(rl) * a.float_pitch) + cl);
        }
    };
    load(0);
    if constexpr (!kDynamic) {
        // the tile's scales: out_scale = FS(scale) leaves right here, the divisor F(FS(scale)) goes to LDS
        const bool rows_fastest = a.sa_row <= a.sa_col;
        for (uint32_t idx = t; idx < kTileRows * bcols; idx += kThreads) {
            const TileScale e = tile_scale<kTileRows>(idx, rows_fastest, bcols_log2);
            const uint32_t gr = place.r0 + e.row, gbc = bc0 + e.bc;
            const bool ok = gr < a.rows && gbc < row_blocks;
            const float s_f = F::round(load_dtype(a.scale_in_dtype, a.scale_in, ok ? gr * a.sa_row + gbc * a.sa_col : 0));
            const float s_fs = round_to_dtype(a.param_dtype, s_f);
            if (ok && a.scale_out != nullptr) store_dtype(a.param_dtype, a.scale_out, gr * a.sb_row + gbc * a.sb_col, s_fs);
            lds_scale[e.row * pitch + e.bc] = F::round(s_fs);
        }
        __syncthreads();
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic

#pragma unroll
    for (int it = 0; it < kIters; it++) {
        if (it + 1 < kIters) {
            load(it + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t tile_row = (it * kUnroll + u) * Shape::kRowWaves + wave_row;
            const uint32_t row = place.r0 + tile_row;
            const bool live = col_live && row < a.rows;
            float v[kN];
            F::unpack(raw[it & 1][u], v);
            float d;
            if constexpr (kDynamic) {
                float amax = 0.0f;
#pragma unroll
                for (int k = 0; k < kN; k++) amax = fmaxf(amax, fabsf(v[k]));  // NaN elements drop out
                amax = group_max_rt(amax, a.group_log2);
                const float s_fs = round_to_dtype(a.param_dtype, block_scale<F>(amax, qp));
                if ((lane & ((1u << a.group_log2) - 1u)) == 0) lds_scale[tile_row * pitch + (tile_chunk >> a.group_log2)] = s_fs;
                d = F::round(s_fs);
            } else {
                d = lds_scale[tile_row * pitch + (tile_chunk >> a.group_log2)];
            }
            uint32_t w[2];
            quantize_chunk<F, kBits, kEnc>(v, d, divisor_is_tame(d), qp, w);
            char* const out_row = out + static_cast<uint64_t>(row) * a.stored_pitch;
            uint32_t* const image_row = lds_words + tile_row * kWordPitch;
            if constexpr (kChunkBits == 64) {
                if constexpr (kStageCodes)
                    image_row[2 * tile_chunk] = w[0], image_row[2 * tile_chunk + 1] = w[1];
                else if (live)
                    stream_store(u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(out_row) + c);
            } else if constexpr (kChunkBits == 32) {
                if constexpr (kStageCodes)
                    image_row[tile_chunk] = w[0];
                else if (live)
                    stream_store(w[0], reinterpret_cast<uint32_t*>(out_row) + c);
            } else {
                constexpr int kLanesPerWord = 32 / kChunkBits;  // 2 or 4: rows are whole words
                const uint32_t sub = lane & (kLanesPerWord - 1);
                const uint32_t word = group_or<kLanesPerWord>(w[0] << (sub * kChunkBits));
                if constexpr (kStageCodes) {
                    if (sub == 0) image_row[tile_chunk / kLanesPerWord] = word;
                } else if (live && sub == 0) {
                    stream_store(word, reinterpret_cast<uint32_t*>(out_row) + c / kLanesPerWord);
                }
            }
        }
    }
    if constexpr (kDynamic || kStageCodes) __syncthreads();
    if constexpr (kStageCodes) {
        const uint32_t w0 = place.c0 * kChunkBits / 32, row_words = a.row_chunks * kChunkBits / 32;
        const uint64_t pitch_words = a.stored_pitch / 4;
        const bool rows_fastest = pitch_words <= a.stored_col;
        for (uint32_t idx = t; idx < kTileRows * kTileWords; idx += kThreads) {
            const TileWord e = tile_word<kTileRows, kTileWords>(idx, rows_fastest);
            const uint32_t gr = place.r0 + e.row, gw = w0 + e.wc;
            if (gr < a.rows && gw < row_words)
                stream_store(lds_words[e.row * kWordPitch + e.wc], reinterpret_cast<uint32_t*>(out) + gr * pitch_words + gw * a.stored_col);
        }
    }
    if constexpr (kDynamic) {
        const bool rows_fastest = a.sb_row <= a.sb_col;
        for (uint32_t idx = t; idx < kTileRows * bcols; idx += kThreads) {
            const TileScale e = tile_scale<kTileRows>(idx, rows_fastest, bcols_log2);
            const uint32_t gr = place.r0 + e.row, gbc = bc0 + e.bc;
            if (gr < a.rows && gbc < row_blocks)
                store_dtype(a.param_dtype, a.scale_out, gr * a.sb_row + gbc * a.sb_col, lds_scale[e.row * pitch + e.bc]);
        }
    }
}

template <class F, int kBits, int kEnc, class Shape, bool kStageCodes>
__global__ __launch_bounds__(kThreads) void dequantize_scale_tiles_kernel(ScaleTileArgs a, uint32_t col_tiles, uint32_t ct_magic,
                                                                         uint32_t ct_shift) {
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    constexpr int kUnroll = Shape::kUnroll, kIters = Shape::kIters, kTileRows = Shape::kTileRows;
    constexpr int kTileWords = Shape::kTileChunks * kChunkBits / 32, kWordPitch = kTileWords + 1;
    extern __shared__ float lds_scale[];
    const uint32_t t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
    const uint32_t wave_row = wave / Shape::kColWaves, tile_chunk = (wave % Shape::kColWaves) * kWave + lane;
    const TilePlace place = tile_place<Shape>(col_tiles, ct_magic, ct_shift);
    const uint32_t bcols_log2 = Shape::kTileChunksLog2 - a.group_log2, bcols = 1u << bcols_log2, pitch = bcols + 1;
    const uint32_t bc0 = place.c0 >> a.group_log2, row_blocks = a.row_chunks >> a.group_log2;
    const uint32_t c = place.c0 + tile_chunk;
    const bool col_live = c < a.row_chunks;
    const uint32_t cl = col_live ? c : a.row_chunks - 1;
    const char* const in = static_cast<const char*>(a.input);
    char* const out = static_cast<char*>(a.output);

    [[maybe_unused]] uint32_t* const lds_words = reinterpret_cast<uint32_t*>(lds_scale + kTileRows * pitch);
    // the loads of iteration it + 1 go out before the arithmetic of iteration it
    uint32_t w0[2][kUnroll], w1[2][kUnroll];
    const auto load = [&](int it) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t tile_row = (it * kUnroll + u) * Shape::kRowWaves + wave_row;
            const uint32_t row = place.r0 + tile_row;
            const char* const in_row = in + static_cast<uint64_t>(row < a.rows ? row : a.rows - 1) * a.stored_pitch;
            w1[it & 1][u] = 0;
            if constexpr (kStageCodes) {  // out of the tile's image in LDS (after the barrier below)
                const uint32_t* const image_row = lds_words + tile_row * kWordPitch;
                if constexpr (kChunkBits == 64)
                    w0[it & 1][u] = image_row[2 * tile_chunk], w1[it & 1][u] = image_row[2 * tile_chunk + 1];
                else if constexpr (kChunkBits == 32)
                    w0[it & 1][u] = image_row[tile_chunk];
                else
                    w0[it & 1][u] = image_row[tile_chunk / (32 / kChunkBits)];
            } else if constexpr (kChunkBits == 64) {
                const u32x2 w = stream_load(reinterpret_cast<const u32x2*>(in_row) + cl);
                w0[it & 1][u] = w[0];
                w1[it & 1][u] = w[1];
            } else if constexpr (kChunkBits == 32) {
                w0[it & 1][u] = stream_load(reinterpret_cast<const uint32_t*>(in_row) + cl);
            } else {
                constexpr int kLanesPerWord = 32 / kChunkBits;
                w0[it & 1][u] = reinterpret_cast<const uint32_t*>(in_row)[cl / kLanesPerWord];  // neighbouring lanes share the word
            }
        }
    };
    if constexpr (kStageCodes) {
        // the tile's words, read along the dimension that is closer in memory in the stored tensor
        const uint32_t word0 = place.c0 * kChunkBits / 32, row_words = a.row_chunks * kChunkBits / 32;
        const uint64_t pitch_words = a.stored_pitch / 4;
        const bool rows_fastest = pitch_words <= a.stored_col;
        for (uint32_t idx = t; idx < kTileRows * kTileWords; idx += kThreads) {
            const TileWord e = tile_word<kTileRows, kTileWords>(idx, rows_fastest);
            const uint32_t gr = place.r0 + e.row, gw = word0 + e.wc;
            const bool ok = gr < a.rows && gw < row_words;
            lds_words[e.row * kWordPitch + e.wc] = stream_load(reinterpret_cast<const uint32_t*>(in) + (ok ? gr * pitch_words + gw * a.stored_col : 0));
        }
    } else {
        load(0);
    }
    {
        const bool rows_fastest = a.sa_row <= a.sa_col;
        for (uint32_t idx = t; idx < kTileRows * bcols; idx += kThreads) {
            const TileScale e = tile_scale<kTileRows>(idx, rows_fastest, bcols_log2);
            const uint32_t gr = place.r0 + e.row, gbc = bc0 + e.bc;
            const bool ok = gr < a.rows && gbc < row_blocks;
            // Line::cast_from(scale)
            lds_scale[e.row * pitch + e.bc] = F::round(load_dtype(a.param_dtype, a.scale_in, ok ? gr * a.sa_row + gbc * a.sa_col : 0));
        }
        __syncthreads();
    }
    if constexpr (kStageCodes) load(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it = 0; it < kIters; it++) {
        if (it + 1 < kIters) {
            load(it + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t tile_row = (it * kUnroll + u) * Shape::kRowWaves + wave_row;
            const uint32_t row = place.r0 + tile_row;
            const float sc = lds_scale[tile_row * pitch + (tile_chunk >> a.group_log2)];
            float y[kN];
            if constexpr (kChunkBits == 64) {
                decode_fields<kEnc, kBits, 4>(w0[it & 1][u], y);
                decode_fields<kEnc, kBits, 4>(w1[it & 1][u], y + 4);
            } else if constexpr (kChunkBits == 32) {
                decode_fields<kEnc, kBits, kN>(w0[it & 1][u], y);
            } else {
                constexpr int kLanesPerWord = 32 / kChunkBits;
                decode_fields<kEnc, kBits, kN>(w0[it & 1][u] >> ((cl & (kLanesPerWord - 1)) * kChunkBits), y);
            }
#pragma unroll
            for (int i = 0; i < kN; i++) y[i] = sc * y[i];
            if (col_live && row < a.rows)
                stream_store(F::pack(y), reinterpret_cast<u32x4*>(out + static_cast<uint64_t>(row) * a.float_pitch) + c);  // pack rounds to F
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
// the stored encodings: kB bits per value, kE the encoding; value ranges wider than their field never come here
#define CQ_SWITCH_STORED(BITS, ENC, ...)                                                              \
    switch (ENC) {                                                                                    \
        case kEncInt:                                                                                 \
            if (BITS == 2) { constexpr int kB = 2; constexpr int kE = kEncInt; __VA_ARGS__; }         \
            if (BITS == 4) { constexpr int kB = 4; constexpr int kE = kEncInt; __VA_ARGS__; }         \
            if (BITS == 8) { constexpr int kB = 8; constexpr int kE = kEncInt; __VA_ARGS__; }         \
            break;                                                                                    \
        case kEncE4M3: if (BITS == 8) { constexpr int kB = 8; constexpr int kE = kEncE4M3; __VA_ARGS__; } break; \
        case kEncE5M2: if (BITS == 8) { constexpr int kB = 8; constexpr int kE = kEncE5M2; __VA_ARGS__; } break; \
        case kEncE2M1: if (BITS == 4) { constexpr int kB = 4; constexpr int kE = kEncE2M1; __VA_ARGS__; } break; \
    }

constexpr uint32_t kMaxDynamicLds = 64u << 10;  // what a workgroup may ask for without further ado

// waves per workgroup of a pieces launch: as many (4, 2, 1) as fit the LDS with both images
uint32_t pieces_waves(uint32_t per, uint32_t chunk_bytes) {
    for (uint32_t waves = kWaves; waves >= 1; waves /= 2)
        if (waves * kWave * per * (16 + chunk_bytes) <= kMaxDynamicLds) return waves;
    return 0;
}

template <class F, int kBits, int kEnc>
hipError_t quantize_pieces(hipStream_t s, const PiecesArgs& a) {
    constexpr uint32_t kChunkBytes = F::kPerChunk * kBits / 8;
    const uint32_t waves = pieces_waves(a.per, kChunkBytes);
    if (waves == 0) return hipErrorInvalidValue;
    const uint64_t wave_chunks = static_cast<uint64_t>(kWave) * a.per;
    const uint64_t num_waves = (a.num_chunks + wave_chunks - 1) / wave_chunks;
    const uint64_t grid = (num_waves + waves - 1) / waves;
    if (grid >= (1ull << 31)) return hipErrorInvalidValue;
    const uint32_t lds = waves * kWave * a.per * (16 + kChunkBytes);
    const uint32_t wide = (reinterpret_cast<uintptr_t>(a.output) & 15u) == 0 ? 1u : 0u;
    const QuantParams qp = quant_params(a.range);
    if (a.scale_in == nullptr)
        hipLaunchKernelGGL((quantize_pieces_kernel<F, kBits, kEnc, true>), dim3(static_cast<uint32_t>(grid)), dim3(waves * kWave), lds, s,
                           static_cast<const u32x4*>(a.input), static_cast<uint32_t*>(a.output), a.scale_in, a.scale_out,
                           a.num_chunks, a.per, a.group_log2, a.param_dtype, wide, qp);
    else
        hipLaunchKernelGGL((quantize_pieces_kernel<F, kBits, kEnc, false>), dim3(static_cast<uint32_t>(grid)), dim3(waves * kWave), lds, s,
                           static_cast<const u32x4*>(a.input), static_cast<uint32_t*>(a.output), a.scale_in, a.scale_out,
                           a.num_chunks, a.per, a.group_log2, a.param_dtype, wide, qp);
    return hipGetLastError();
}

struct TileGrid {
    uint32_t grid, col_tiles, magic, shift, lds;
    bool ok;
};
template <class Shape>
TileGrid tile_grid(const ScaleTileArgs& a) {
    TileGrid g{};
    g.col_tiles = (a.row_chunks + Shape::kTileChunks - 1) / Shape::kTileChunks;
    const uint64_t tiles = static_cast<uint64_t>((a.rows + Shape::kTileRows - 1) / Shape::kTileRows) * g.col_tiles;
    g.ok = tiles < (1ull << 31);
    g.grid = static_cast<uint32_t>(tiles);
    magic_of(g.col_tiles, &g.magic, &g.shift);
    g.lds = Shape::kTileRows * ((Shape::kTileChunks >> a.group_log2) + 1) * static_cast<uint32_t>(sizeof(float));
    return g;
}
// LDS of the image of a tile's words (staged codes)
template <class Shape>
uint32_t tile_words_lds(uint32_t chunk_bits) {
    return Shape::kTileRows * (Shape::kTileChunks * chunk_bits / 32 + 1) * 4u;
}

template <class F, int kBits, int kEnc, class Shape, bool kStageCodes>
hipError_t quantize_scale_tiles_shape(hipStream_t s, const ScaleTileArgs& a) {
    const TileGrid g = tile_grid<Shape>(a);
    if (!g.ok) return hipErrorInvalidValue;
    const QuantParams qp = quant_params(a.range);
    const uint32_t lds = g.lds + (kStageCodes ? tile_words_lds<Shape>(F::kPerChunk * kBits) : 0u);
    if (a.scale_in == nullptr)
        hipLaunchKernelGGL((quantize_scale_tiles_kernel<F, kBits, kEnc, true, Shape, kStageCodes>), dim3(g.grid), dim3(kThreads), lds, s,
                           a, qp, g.col_tiles, g.magic, g.shift);
    else
        hipLaunchKernelGGL((quantize_scale_tiles_kernel<F, kBits, kEnc, false, Shape, kStageCodes>), dim3(g.grid), dim3(kThreads), lds, s,
                           a, qp, g.col_tiles, g.magic, g.shift);
    return hipGetLastError();
}
template <class F, int kBits, int kEnc, class Shape, bool kStageCodes>
hipError_t dequantize_scale_tiles_shape(hipStream_t s, const ScaleTileArgs& a) {
    const TileGrid g = tile_grid<Shape>(a);
    if (!g.ok) return hipErrorInvalidValue;
    const uint32_t lds = g.lds + (kStageCodes ? tile_words_lds<Shape>(F::kPerChunk * kBits) : 0u);
    hipLaunchKernelGGL((dequantize_scale_tiles_kernel<F, kBits, kEnc, Shape, kStageCodes>), dim3(g.grid), dim3(kThreads), lds, s, a,
                       g.col_tiles, g.magic, g.shift);
    return hipGetLastError();
}

// Tiles of 16 rows x 64 chunks, four steps in flight and no loop: measured on bf16 [28672, 8192] with 4-bit codes on
// blocks of 32 and scales stored column by column against tiles of 32 rows in two or four iterations (given scales
// 102 us against 112 us, dequantize 95 us against 119 us), tiles of 256 chunks (104 - 116 us) and tiles of 8 rows
// (107 us / 96 us).
using QuantizeTile = TileShape<16, 1, 4>;
using DequantizeTile = TileShape<16, 1, 4>;
// Staged codes (a stored tensor whose last dimension is not the contiguous one; words of the U32 store only): 32 rows,
// so that the runs along the rows are whole 128-byte lines
using StagedCodesTile = TileShape<32, 1, 4>;

template <class F, int kBits, int kEnc>
hipError_t quantize_scale_tiles(hipStream_t s, const ScaleTileArgs& a) {
    if (a.stored_col != 1) {
        if constexpr (kEnc == kEncInt)
            return quantize_scale_tiles_shape<F, kBits, kEnc, StagedCodesTile, true>(s, a);
        else
            return hipErrorInvalidValue;
    }
    return quantize_scale_tiles_shape<F, kBits, kEnc, QuantizeTile, false>(s, a);
}

template <class F, int kBits, int kEnc>
hipError_t dequantize_scale_tiles(hipStream_t s, const ScaleTileArgs& a) {
    if (a.stored_col != 1) {
        if constexpr (kEnc == kEncInt)
            return dequantize_scale_tiles_shape<F, kBits, kEnc, StagedCodesTile, true>(s, a);
        else
            return hipErrorInvalidValue;
    }
    return dequantize_scale_tiles_shape<F, kBits, kEnc, DequantizeTile, false>(s, a);
}

}  // namespace

// Blocks of `block` values as pieces: a whole number of chunks that is not a power of two up to 32 (those are
// the flat kernels'), its odd factor small enough for the LDS of at least one wave.
bool pieces_supported(int dtype, int bits, uint32_t block, uint32_t* per, uint32_t* group_log2) {
    const uint32_t per_chunk = dtype == CQ_F32 ? 4u : 8u;
    if (block == 0 || block % per_chunk != 0) return false;
    uint32_t g = block / per_chunk, log2 = 0;
    while (g % 2 == 0) {
        g /= 2;
        log2++;
    }
    if (g == 1 || log2 > 6) return false;
    if (pieces_waves(g, per_chunk * static_cast<uint32_t>(bits) / 8) == 0) return false;
    *per = g;
    *group_log2 = log2;
    return true;
}

hipError_t launch_quantize_pieces(hipStream_t s, int dtype, int bits, const PiecesArgs& a) {
    if (a.num_chunks == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_STORED(bits, a.encoding, return (quantize_pieces<kF, kB, kE>(s, a))) break)
    return hipErrorInvalidValue;
}

hipError_t launch_quantize_scale_tiles(hipStream_t s, int dtype, int bits, const ScaleTileArgs& a) {
    if (a.rows == 0 || a.row_chunks == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_STORED(bits, a.encoding, return (quantize_scale_tiles<kF, kB, kE>(s, a))) break)
    return hipErrorInvalidValue;
}

hipError_t launch_dequantize_scale_tiles(hipStream_t s, int dtype, int bits, const ScaleTileArgs& a) {
    if (a.rows == 0 || a.row_chunks == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, CQ_SWITCH_STORED(bits, a.encoding, return (dequantize_scale_tiles<kF, kB, kE>(s, a))) break)
    return hipErrorInvalidValue;
}

}  // namespace cq
