// Abs-max along one axis: out[.., 0, ..] = max_k |in[.., k, ..]|, the MaxAbs
// reduction a caller of the reference runs in front of quantize to build scales
// (crates/cubek-reduce/src/instructions/maxabs.rs:47-96, entry point
// crates/cubek-reduce/src/lib.rs:93-131).  NaN elements are ignored; abs and max
// are exact, so any evaluation order gives the same bits.
//
// A contiguous tensor is viewed as [outer, L, inner] around the reduced axis.
//   inner == 1 (innermost axis):  rows of L contiguous elements
//        rows that are 1..64 chunks long (power of two): lane groups + DPP butterfly
//        otherwise one wave per (row, slice) with 16-byte lane-strided loads
//   inner a multiple of one 16-byte chunk:
//        wide or many: one lane per (outer, inner chunk) walking L with stride `inner`
//        narrow, few:  one workgroup per (outer, tile of chunk columns, slice of L);
//                      its lanes form a [row phase][chunk column] grid, so a step
//                      reads whole rows of the tile, and combine through LDS
// When the outputs alone give too few workgroups to fill the GPU, L is cut into
// slices whose f32 partial maxima go to a caller-provided workspace
// ([slice][output]) and a second kernel folds them (the same tile kernel over the
// partials).  Anything else (strided tensors, odd inner sizes) takes a
// one-wave-per-output (long axis) or one-thread-per-output fallback.
#include "cq_device.hpp"
#include "cq_internal.hpp"
#include "cq_magic_div.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;

template <class F>
__device__ __forceinline__ float chunk_absmax(u32x4 raw, float acc) {
    float v[F::kPerChunk];
    F::unpack(raw, v);
#pragma unroll
    for (int i = 0; i < F::kPerChunk; i++) acc = fmaxf(acc, fabsf(v[i]));
    return acc;
}

// ---- rows, short: kGroup lanes per row ---------------------------------------
template <class F, int kGroup, int kUnroll>
__global__ __launch_bounds__(kThreads) void reduce_rows_grouped_kernel(const u32x4* __restrict__ in,
                                                                       void* __restrict__ out,
                                                                       uint64_t num_chunks) {
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
    u32x4 raw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        raw[u] = stream_load(in + (c < num_chunks ? c : num_chunks - 1));
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float amax = group_max<kGroup>(chunk_absmax<F>(raw[u], 0.0f));
        if (c < num_chunks && (c % kGroup) == 0) F::store(out, c / kGroup, amax);
    }
}

// ---- rows, long: one wave per (row, slice) --------------------------------------
// kPartial: write f32 partials [slice][row] with row pitch `pitch`; otherwise the
// final value typed F.
template <class F, bool kPartial>
__global__ __launch_bounds__(kThreads) void reduce_rows_wave_kernel(const u32x4* __restrict__ in,
                                                                    void* __restrict__ out, uint64_t rows,
                                                                    uint64_t chunks_per_row, uint32_t slices,
                                                                    uint64_t pitch) {
    constexpr int kUnroll = 4;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint64_t job = static_cast<uint64_t>(blockIdx.x) * (kThreads / kWave) + threadIdx.x / kWave;
    if (job >= rows * slices) return;  // whole waves leave together
    const uint64_t row = job / slices;
    const uint32_t slice = static_cast<uint32_t>(job % slices);
    const uint64_t per_slice = (chunks_per_row + slices - 1) / slices;
    const uint64_t begin = slice * per_slice;
    const uint64_t end = begin + per_slice < chunks_per_row ? begin + per_slice : chunks_per_row;
    const u32x4* p = in + row * chunks_per_row;
    float amax = 0.0f;
    for (uint64_t c0 = begin + lane; c0 < end; c0 += kWave * kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t c = c0 + static_cast<uint64_t>(u) * kWave;
            raw[u] = stream_load(p + (c < end ? c : end - 1));  // re-reading a chunk is harmless for max
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) amax = chunk_absmax<F>(raw[u], amax);
    }
    amax = group_max<64>(amax);
    if (lane == 0) {
        if constexpr (kPartial)
            static_cast<float*>(out)[static_cast<uint64_t>(slice) * pitch + row] = amax;
        else
            F::store(out, row, amax);
    }
}

// ---- columns, wide: one lane per (slice of L, outer, inner chunk) ---------------------
// kPartial: write f32 partials [slice][output]; otherwise the final chunk typed F.
template <class F, bool kPartial>
__global__ __launch_bounds__(kThreads) void reduce_cols_kernel(const u32x4* __restrict__ in, void* __restrict__ out,
                                                               uint64_t outer, uint64_t len, uint64_t inner_chunks,
                                                               uint32_t slices) {
    constexpr int kN = F::kPerChunk;
    constexpr int kUnroll = 4;
    const uint64_t cols = outer * inner_chunks;  // output chunks
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (t >= cols * slices) return;
    const uint32_t slice = static_cast<uint32_t>(t / cols);
    const uint64_t col = t % cols;
    const uint64_t o = col / inner_chunks, j = col % inner_chunks;
    const uint64_t per_slice = (len + slices - 1) / slices;
    const uint64_t begin = slice * per_slice;
    const uint64_t end = begin + per_slice < len ? begin + per_slice : len;
    const u32x4* p = in + o * len * inner_chunks + j;
    float amax[kN];
#pragma unroll
    for (int i = 0; i < kN; i++) amax[i] = 0.0f;
    for (uint64_t l0 = begin; l0 < end; l0 += kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t l = l0 + u < end ? l0 + u : end - 1;
            raw[u] = stream_load(p + l * inner_chunks);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            float v[kN];
            F::unpack(raw[u], v);
#pragma unroll
            for (int i = 0; i < kN; i++) amax[i] = fmaxf(amax[i], fabsf(v[i]));
        }
    }
    if constexpr (kPartial) {
        float* dst = static_cast<float*>(out) + (static_cast<uint64_t>(slice) * cols + col) * kN;
#pragma unroll
        for (int i = 0; i < kN; i++) dst[i] = amax[i];
    } else {
        static_cast<u32x4*>(out)[col] = F::pack(amax);  // values are F numbers: packing is exact
    }
}

// ---- columns, few outputs: one workgroup per (outer, column tile, slice of L) ----------
// Lanes form a [kT / kCW row phases][kCW chunk columns] grid.  FIn is the type read
// (F32 when folding partials), FOut the type of the final result.
enum TileOut { kTileFinalPacked = 0, kTilePartial = 1, kTileFinalChecked = 2 };

template <class FIn, class FOut, int kCW, int kT, int kMode>
__global__ __launch_bounds__(kT) void reduce_tile_kernel(const u32x4* __restrict__ in, void* __restrict__ out,
                                                         uint64_t len, uint64_t inner_chunks, uint32_t col_tiles,
                                                         uint32_t slices, uint64_t pitch, uint64_t count) {
    static_assert(kCW >= 1 && kCW <= kWave && kT % kWave == 0, "a tile row fits in one wave");
    constexpr int kN = FIn::kPerChunk;
    constexpr int kRH = kT / kCW;
    constexpr int kUnroll = 4;
    constexpr int kWaves = kT / kWave;
    const uint64_t job = blockIdx.x;
    // column tiles vary fastest: workgroups in flight together read whole rows, which
    // spreads their requests over all memory channels
    const uint32_t tile = static_cast<uint32_t>(job % col_tiles);
    const uint32_t slice = static_cast<uint32_t>((job / col_tiles) % slices);
    const uint64_t o = job / col_tiles / slices;
    const uint32_t cx = threadIdx.x % kCW, ry = threadIdx.x / kCW;
    const uint64_t j = static_cast<uint64_t>(tile) * kCW + cx;
    const uint64_t per_slice = (len + slices - 1) / slices;
    const uint64_t begin = slice * per_slice;
    const uint64_t end = begin + per_slice < len ? begin + per_slice : len;
    const u32x4* p = in + o * len * inner_chunks + (j < inner_chunks ? j : inner_chunks - 1);
    float amax[kN];
#pragma unroll
    for (int i = 0; i < kN; i++) amax[i] = 0.0f;
    for (uint64_t l0 = begin + ry; l0 < end; l0 += kRH * kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t l = l0 + static_cast<uint64_t>(u) * kRH;
            raw[u] = stream_load(p + (l < end ? l : end - 1) * inner_chunks);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            float v[kN];
            FIn::unpack(raw[u], v);
#pragma unroll
            for (int i = 0; i < kN; i++) amax[i] = fmaxf(amax[i], fabsf(v[i]));
        }
    }
    // lanes of a wave that share a column
#pragma unroll
    for (int mask = kCW; mask < kWave; mask <<= 1) {
#pragma unroll
        for (int i = 0; i < kN; i++) amax[i] = fmaxf(amax[i], __shfl_xor(amax[i], mask, kWave));
    }
    __shared__ float lds[kWaves][kCW][kN];
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane < kCW) {
#pragma unroll
        for (int i = 0; i < kN; i++) lds[wave][lane][i] = amax[i];
    }
    __syncthreads();
    if (threadIdx.x >= kCW || j >= inner_chunks) return;
#pragma unroll
    for (int w = 1; w < kWaves; w++) {
#pragma unroll
        for (int i = 0; i < kN; i++) amax[i] = fmaxf(amax[i], lds[w][cx][i]);
    }
    const uint64_t col = o * inner_chunks + j;
    if constexpr (kMode == kTilePartial) {
        float* dst = static_cast<float*>(out) + static_cast<uint64_t>(slice) * pitch + col * kN;
#pragma unroll
        for (int i = 0; i < kN; i++) dst[i] = amax[i];
    } else if constexpr (kMode == kTileFinalPacked) {
        static_cast<u32x4*>(out)[col] = FOut::pack(amax);
    } else {
#pragma unroll
        for (int i = 0; i < kN; i++)
            if (col * kN + i < count) FOut::store(out, col * kN + i, amax[i]);
    }
}

// ---- strided inputs with a contiguous last dimension ------------------------------------
// The dimensions that are not reduced, innermost first (`count` entries each, multiply-and-shift
// divisions), with their input strides in 32-bit words (rows start on multiples of 4 bytes; the 16-byte
// loads then sit off their natural alignment, which the hardware takes); the outputs are contiguous.
struct ReduceLevels {
    uint32_t levels;
    uint32_t count[CQ_MAX_RANK], magic[CQ_MAX_RANK], shift[CQ_MAX_RANK];
    uint64_t in[CQ_MAX_RANK];
};
__device__ __forceinline__ uint64_t level_offset(const ReduceLevels& r, uint32_t n) {
    uint64_t off = 0;
#pragma unroll
    for (int l = 0; l < CQ_MAX_RANK; l++) {
        if (l < static_cast<int>(r.levels)) {
            uint32_t index = n;
            if (l + 1 < static_cast<int>(r.levels)) {
                const uint32_t q = magic_div(n, r.magic[l], r.shift[l]);
                index = n - q * r.count[l];
                n = q;
            }
            off += index * r.in[l];
        }
    }
    return off;
}

__device__ __forceinline__ const u32x4* words_at(const u32x4* base, uint64_t words) {
    return reinterpret_cast<const u32x4*>(reinterpret_cast<const uint32_t*>(base) + words);
}

// reduce_rows_grouped_kernel with the rows (all dimensions but the last) found through `r`
template <class F, int kGroup, int kUnroll>
__global__ __launch_bounds__(kThreads) void reduce_rows_grouped_strided_kernel(const u32x4* __restrict__ in,
                                                                               void* __restrict__ out, ReduceLevels r,
                                                                               uint64_t num_chunks) {
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
    u32x4 raw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        c = c < num_chunks ? c : num_chunks - 1;
        raw[u] = stream_load(words_at(in, level_offset(r, static_cast<uint32_t>(c / kGroup))) + c % kGroup);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float amax = group_max<kGroup>(chunk_absmax<F>(raw[u], 0.0f));
        if (c < num_chunks && (c % kGroup) == 0) F::store(out, c / kGroup, amax);
    }
}

// reduce_rows_wave_kernel with the rows found through `r`
template <class F, bool kPartial>
__global__ __launch_bounds__(kThreads) void reduce_rows_wave_strided_kernel(const u32x4* __restrict__ in,
                                                                            void* __restrict__ out, ReduceLevels r,
                                                                            uint64_t rows, uint64_t chunks_per_row,
                                                                            uint32_t slices, uint64_t pitch) {
    constexpr int kUnroll = 4;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint64_t job = static_cast<uint64_t>(blockIdx.x) * (kThreads / kWave) + threadIdx.x / kWave;
    if (job >= rows * slices) return;  // whole waves leave together
    const uint64_t row = job / slices;
    const uint32_t slice = static_cast<uint32_t>(job % slices);
    const uint64_t per_slice = (chunks_per_row + slices - 1) / slices;
    const uint64_t begin = slice * per_slice;
    const uint64_t end = begin + per_slice < chunks_per_row ? begin + per_slice : chunks_per_row;
    const u32x4* p = words_at(in, level_offset(r, static_cast<uint32_t>(row)));
    float amax = 0.0f;
    for (uint64_t c0 = begin + lane; c0 < end; c0 += kWave * kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t c = c0 + static_cast<uint64_t>(u) * kWave;
            raw[u] = stream_load(p + (c < end ? c : end - 1));
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) amax = chunk_absmax<F>(raw[u], amax);
    }
    amax = group_max<64>(amax);
    if (lane == 0) {
        if constexpr (kPartial)
            static_cast<float*>(out)[static_cast<uint64_t>(slice) * pitch + row] = amax;
        else
            F::store(out, row, amax);
    }
}

// reduce_cols_kernel with the output chunks (the last dimension in chunks, then the other kept
// dimensions) found through `r`; the reduced axis steps `len_stride` words
template <class F, bool kPartial>
__global__ __launch_bounds__(kThreads) void reduce_cols_strided_kernel(const u32x4* __restrict__ in, void* __restrict__ out,
                                                                       ReduceLevels r, uint64_t cols, uint64_t len,
                                                                       uint64_t len_stride, uint32_t slices) {
    constexpr int kN = F::kPerChunk;
    constexpr int kUnroll = 4;
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (t >= cols * slices) return;
    const uint32_t slice = static_cast<uint32_t>(t / cols);
    const uint64_t col = t % cols;
    const uint64_t per_slice = (len + slices - 1) / slices;
    const uint64_t begin = slice * per_slice;
    const uint64_t end = begin + per_slice < len ? begin + per_slice : len;
    const u32x4* p = words_at(in, level_offset(r, static_cast<uint32_t>(col)));
    float amax[kN];
#pragma unroll
    for (int i = 0; i < kN; i++) amax[i] = 0.0f;
    for (uint64_t l0 = begin; l0 < end; l0 += kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t l = l0 + u < end ? l0 + u : end - 1;
            raw[u] = stream_load(words_at(p, l * len_stride));
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            float v[kN];
            F::unpack(raw[u], v);
#pragma unroll
            for (int i = 0; i < kN; i++) amax[i] = fmaxf(amax[i], fabsf(v[i]));
        }
    }
    if constexpr (kPartial) {
        float* dst = static_cast<float*>(out) + (static_cast<uint64_t>(slice) * cols + col) * kN;
#pragma unroll
        for (int i = 0; i < kN; i++) dst[i] = amax[i];
    } else {
        static_cast<u32x4*>(out)[col] = F::pack(amax);
    }
}

// ---- fallbacks: any strides -----------------------------------------------------------
struct StridedReduce {
    uint32_t rank, axis;
    uint32_t shape[CQ_MAX_RANK];
    uint64_t in_strides[CQ_MAX_RANK];
    uint64_t out_strides[CQ_MAX_RANK];
};

// kLanes lanes per output element (1 or a whole wave)
template <class F, int kLanes>
__global__ __launch_bounds__(kThreads) void reduce_strided_kernel(const void* __restrict__ in,
                                                                  void* __restrict__ out, StridedReduce r,
                                                                  uint64_t num_out) {
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const uint64_t i = t / kLanes;
    const uint32_t lane = static_cast<uint32_t>(t % kLanes);
    if (i >= num_out) return;  // kLanes divides the wave: whole groups leave together
    uint64_t rem = i, in_off = 0, out_off = 0;
    for (int d = static_cast<int>(r.rank) - 1; d >= 0; d--) {
        if (static_cast<uint32_t>(d) == r.axis) continue;
        const uint64_t c = rem % r.shape[d];
        rem /= r.shape[d];
        in_off += c * r.in_strides[d];
        out_off += c * r.out_strides[d];
    }
    float m = 0.0f;
    for (uint32_t k = lane; k < r.shape[r.axis]; k += kLanes)
        m = fmaxf(m, fabsf(F::load(in, in_off + static_cast<uint64_t>(k) * r.in_strides[r.axis])));
    m = group_max<kLanes>(m);
    if (lane == 0) F::store(out, out_off, m);
}

// Output element i of a contiguous result -> its place in a strided output tensor.
template <class F>
__global__ __launch_bounds__(kThreads) void scatter_outputs_kernel(const void* __restrict__ packed, void* __restrict__ out,
                                                                   StridedReduce r, uint64_t num_out) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (i >= num_out) return;
    uint64_t rem = i, out_off = 0;
    for (int d = static_cast<int>(r.rank) - 1; d >= 0; d--) {
        if (static_cast<uint32_t>(d) == r.axis) continue;
        const uint64_t c = rem % r.shape[d];
        rem /= r.shape[d];
        out_off += c * r.out_strides[d];
    }
    if constexpr (F::kBytes == 4)
        static_cast<uint32_t*>(out)[out_off] = static_cast<const uint32_t*>(packed)[i];
    else
        static_cast<uint16_t*>(out)[out_off] = static_cast<const uint16_t*>(packed)[i];
}

// bytes of the workspace that hold the contiguous result of a launch whose output tensor is strided
inline uint64_t packed_outputs_bytes(uint64_t num_out, uint64_t elem_bytes) { return (num_out * elem_bytes + 255) / 256 * 256; }

inline dim3 blocks(uint64_t n, uint64_t per_block) { return dim3(static_cast<uint32_t>((n + per_block - 1) / per_block)); }
inline uint64_t round_up(uint64_t v, uint64_t m) { return (v + m - 1) / m * m; }
inline uint32_t pow2_at_least(uint64_t v, uint32_t cap) {
    uint32_t p = 1;
    while (p < v && p < cap) p <<= 1;
    return p;
}

// enough workgroups / lanes to keep 256 CUs busy
constexpr uint64_t kTargetGroups = 2048;
constexpr uint64_t kTargetLanes = kTargetGroups * kThreads / 2;

// How a contiguous [outer, len, inner] view is cut up; shared by the launcher and
// by the workspace size query so that the two always agree.
struct ReducePlan {
    enum Kind { kFallback, kRowsGrouped, kRowsWave, kCols, kTile } kind = kFallback;
    uint64_t chunks_per_row = 0, inner_chunks = 0;
    uint32_t cw = 1, col_tiles = 1;
    uint64_t slices = 1;  // wanted; the launcher lowers it to what the workspace holds
    uint64_t lane_slices = 1;  // kTile on a strided input (one lane per output chunk and slice instead): wanted there
    uint64_t pitch = 0;   // floats per slice of partials
};

ReducePlan plan_reduce(uint64_t outer, uint64_t len, uint64_t inner, uint64_t kN) {
    ReducePlan p;
    // partials (f32 per output and slice) stay below 1/32 of the bytes read
    const uint64_t traffic_cap = len * (16 / kN) / 128 > 0 ? len * (16 / kN) / 128 : 1;
    if (len == 0 || outer == 0 || inner == 0) return p;
    if (inner == 1 && len % kN == 0) {
        p.chunks_per_row = len / kN;
        if (p.chunks_per_row <= 64 && (p.chunks_per_row & (p.chunks_per_row - 1)) == 0) {
            p.kind = ReducePlan::kRowsGrouped;
            return p;
        }
        p.kind = ReducePlan::kRowsWave;
        p.pitch = round_up(outer, 4);
        if (outer * kWave < kTargetLanes) {
            p.slices = kTargetLanes / (outer * kWave);
            const uint64_t max_slices = (p.chunks_per_row + 8 * kWave - 1) / (8 * kWave);  // >= 8 KiB per wave and slice
            if (p.slices > max_slices) p.slices = max_slices;
            if (p.slices > traffic_cap) p.slices = traffic_cap;
        }
        return p;
    }
    if (inner % kN != 0) return p;
    p.inner_chunks = inner / kN;
    const uint64_t cols = outer * p.inner_chunks;
    if (cols >= kTargetLanes || p.inner_chunks >= kThreads) {
        p.kind = ReducePlan::kCols;
        p.pitch = outer * inner;
        if (cols < kTargetLanes) {
            p.slices = kTargetLanes / cols;
            const uint64_t max_slices = (len + 15) / 16;  // at least 16 rows per slice
            if (p.slices > max_slices) p.slices = max_slices;
            if (p.slices > traffic_cap) p.slices = traffic_cap;
        }
        return p;
    }
    p.kind = ReducePlan::kTile;
    p.lane_slices = kTargetLanes / cols;
    if (p.lane_slices > (len + 15) / 16) p.lane_slices = (len + 15) / 16;
    if (p.lane_slices > traffic_cap) p.lane_slices = traffic_cap;
    if (p.lane_slices < 1) p.lane_slices = 1;
    p.cw = pow2_at_least(p.inner_chunks, kWave);
    p.col_tiles = static_cast<uint32_t>((p.inner_chunks + p.cw - 1) / p.cw);
    p.pitch = outer * inner;  // a multiple of kN, hence of 4
    const uint64_t base = outer * p.col_tiles;
    if (base < kTargetGroups) {
        p.slices = kTargetGroups / base;
        const uint64_t rows_per_step = kThreads / p.cw * 4;  // rows one workgroup reads per loop trip
        const uint64_t max_slices = (len + 2 * rows_per_step - 1) / (2 * rows_per_step);
        if (p.slices > max_slices) p.slices = max_slices;
        if (p.slices > traffic_cap) p.slices = traffic_cap;
    }
    return p;
}

template <class FIn, class FOut, int kT, int kMode>
void launch_tile(hipStream_t s, uint32_t cw, uint64_t jobs, const void* in, void* out, uint64_t len,
                 uint64_t inner_chunks, uint32_t col_tiles, uint32_t slices, uint64_t pitch, uint64_t count) {
    auto src = static_cast<const u32x4*>(in);
    dim3 grid(static_cast<uint32_t>(jobs));
    switch (cw) {
#define CQ_CASE(W) case W: hipLaunchKernelGGL((reduce_tile_kernel<FIn, FOut, W, kT, kMode>), grid, dim3(kT), 0, s, src, out, len, inner_chunks, col_tiles, slices, pitch, count); break;
        CQ_CASE(1) CQ_CASE(2) CQ_CASE(4) CQ_CASE(8) CQ_CASE(16) CQ_CASE(32) CQ_CASE(64)
#undef CQ_CASE
    }
}

// out[i] = max_s partials[s][i], i < count; partials are f32 with row pitch `pitch`
template <class F>
void launch_fold(hipStream_t s, const void* partials, void* out, uint64_t slices, uint64_t pitch, uint64_t count) {
    constexpr int kFoldThreads = 1024;
    const uint64_t chunks = pitch / 4;
    uint32_t cw = pow2_at_least(chunks, kWave);
    while (cw > 4 && chunks / cw < 128) cw /= 2;  // narrower tiles, more workgroups: the partials sit in L2
    const uint32_t tiles = static_cast<uint32_t>((chunks + cw - 1) / cw);
    launch_tile<F32, F, kFoldThreads, kTileFinalChecked>(s, cw, tiles, partials, out, slices, chunks, tiles, 1u, 0, count);
}

// The levels of a strided input with a contiguous last dimension of whole chunks, strides of whole words and
// fewer than 2^31 rows and output chunks; false: not such a tensor.
template <class F>
bool strided_levels(const ReduceArgs& a, ReduceLevels* r, uint64_t* len_stride) {
    constexpr uint64_t kN = F::kPerChunk;
    constexpr uint64_t kWordElems = F::kBytes == 4 ? 1 : 2;  // elements per 32-bit word
    if (a.rank < 2 || (reinterpret_cast<uintptr_t>(a.input) & 3u) != 0) return false;
    const uint32_t last = a.rank - 1;
    if (a.in_strides[last] != 1 || a.shape[last] % kN != 0) return false;
    *r = ReduceLevels{};
    *len_stride = 0;
    uint64_t total = 1;
    const auto push = [&](uint64_t count, uint64_t stride) {
        const uint32_t k = r->levels;
        if (k > 0 && stride == r->in[k - 1] * r->count[k - 1] && r->count[k - 1] * count < (1ull << 31)) {
            r->count[k - 1] *= static_cast<uint32_t>(count);  // steps on uniformly from the level inside it
        } else {
            r->count[k] = static_cast<uint32_t>(count);
            r->in[k] = stride;
            r->levels = k + 1;
        }
        total *= count;
    };
    if (a.axis != last) push(a.shape[last] / kN, 4);  // a chunk is four words
    for (int d = static_cast<int>(last) - 1; d >= 0; d--) {
        if (a.in_strides[d] % kWordElems != 0 && a.shape[d] > 1) return false;
        if (static_cast<uint32_t>(d) == a.axis) {
            *len_stride = a.in_strides[d] / kWordElems;
            continue;
        }
        if (a.shape[d] == 1) continue;
        push(a.shape[d], a.in_strides[d] / kWordElems);
    }
    if (r->levels == 0) push(1, 0);
    if (total >= (1ull << 31)) return false;
    for (uint32_t l = 0; l < r->levels; l++) magic_of(r->count[l], &r->magic[l], &r->shift[l]);
    return true;
}

template <class F>
hipError_t reduce_dispatch(hipStream_t s, const ReduceArgs& a) {
    constexpr uint64_t kN = F::kPerChunk;
    // A strided output (one column of a matrix, every other element): the kernels below write a contiguous result
    // into the front of the workspace, and one more small launch puts every element in its place.  Without that much
    // workspace the launch runs one wave (or lane) per output.
    if (!a.out_contiguous) {
        const uint64_t num_out = a.outer * a.inner, front = packed_outputs_bytes(num_out, F::kBytes);
        if (a.workspace != nullptr && a.workspace_bytes >= front && num_out != 0) {
            ReduceArgs b = a;
            b.output = a.workspace;
            b.out_contiguous = true;
            b.contiguous = a.in_contiguous;
            uint64_t acc = 1;
            for (int d = static_cast<int>(a.rank) - 1; d >= 0; d--) {
                b.out_strides[d] = acc;
                if (static_cast<uint32_t>(d) != a.axis) acc *= a.shape[d];
            }
            b.workspace = static_cast<char*>(a.workspace) + front;
            b.workspace_bytes = a.workspace_bytes - front;
            if (b.workspace_bytes == 0) b.workspace = nullptr;
            const hipError_t e = reduce_dispatch<F>(s, b);
            if (e != hipSuccess) return e;
            StridedReduce r{};
            r.rank = a.rank;
            r.axis = a.axis;
            for (uint32_t d = 0; d < a.rank; d++) {
                r.shape[d] = static_cast<uint32_t>(a.shape[d]);
                r.out_strides[d] = a.out_strides[d];
            }
            hipLaunchKernelGGL((scatter_outputs_kernel<F>), blocks(num_out, kThreads), dim3(kThreads), 0, s, a.workspace, a.output, r,
                               num_out);
            return hipGetLastError();
        }
    }
    ReducePlan p;
    if (a.contiguous && (reinterpret_cast<uintptr_t>(a.input) & 15u) == 0) p = plan_reduce(a.outer, a.len, a.inner, kN);
    ReduceLevels levels;
    uint64_t len_stride = 0;
    if (!a.contiguous && a.out_contiguous && strided_levels<F>(a, &levels, &len_stride)) {
        // the plan of the contiguous tensor of this shape, with kernels that look up where rows and columns lie
        p = plan_reduce(a.outer, a.len, a.inner, kN);
        const bool rows = p.kind == ReducePlan::kRowsGrouped || p.kind == ReducePlan::kRowsWave;
        const bool cols = p.kind == ReducePlan::kCols || p.kind == ReducePlan::kTile;
        if ((rows && a.axis != a.rank - 1) || (cols && (a.axis == a.rank - 1 || (reinterpret_cast<uintptr_t>(a.output) & 15u) != 0)))
            p.kind = ReducePlan::kFallback;
        uint64_t slices = p.kind == ReducePlan::kTile ? p.lane_slices : p.slices;
        if (slices > 1) {
            const uint64_t fit = a.workspace == nullptr ? 0 : a.workspace_bytes / (p.pitch * sizeof(float));
            if (slices > fit) slices = fit > 1 ? fit : 1;
        }
        auto in = static_cast<const u32x4*>(a.input);
        if (p.kind == ReducePlan::kRowsGrouped) {
            const uint64_t num_chunks = a.outer * p.chunks_per_row;
            constexpr int kU = 4;
            dim3 grid = blocks(num_chunks, kThreads * kU);
            switch (p.chunks_per_row) {
#define CQ_CASE(G) case G: hipLaunchKernelGGL((reduce_rows_grouped_strided_kernel<F, G, kU>), grid, dim3(kThreads), 0, s, in, a.output, levels, num_chunks); break;
                CQ_CASE(1) CQ_CASE(2) CQ_CASE(4) CQ_CASE(8) CQ_CASE(16) CQ_CASE(32) CQ_CASE(64)
#undef CQ_CASE
            }
            return hipGetLastError();
        }
        if (p.kind == ReducePlan::kRowsWave) {
            dim3 grid = blocks(a.outer * slices, kThreads / kWave);
            if (slices > 1) {
                hipLaunchKernelGGL((reduce_rows_wave_strided_kernel<F, true>), grid, dim3(kThreads), 0, s, in, a.workspace,
                                   levels, a.outer, p.chunks_per_row, static_cast<uint32_t>(slices), p.pitch);
                launch_fold<F>(s, a.workspace, a.output, slices, p.pitch, a.outer);
            } else {
                hipLaunchKernelGGL((reduce_rows_wave_strided_kernel<F, false>), grid, dim3(kThreads), 0, s, in, a.output,
                                   levels, a.outer, p.chunks_per_row, 1u, 0);
            }
            return hipGetLastError();
        }
        if (cols && p.kind != ReducePlan::kFallback) {
            const uint64_t out_chunks = a.outer * p.inner_chunks;
            dim3 grid = blocks(out_chunks * slices, kThreads);
            if (slices > 1) {
                hipLaunchKernelGGL((reduce_cols_strided_kernel<F, true>), grid, dim3(kThreads), 0, s, in, a.workspace, levels,
                                   out_chunks, a.len, len_stride, static_cast<uint32_t>(slices));
                launch_fold<F>(s, a.workspace, a.output, slices, p.pitch, p.pitch);
            } else {
                hipLaunchKernelGGL((reduce_cols_strided_kernel<F, false>), grid, dim3(kThreads), 0, s, in, a.output, levels,
                                   out_chunks, a.len, len_stride, 1u);
            }
            return hipGetLastError();
        }
        p = ReducePlan{};
    }
    if ((p.kind == ReducePlan::kCols || p.kind == ReducePlan::kTile) && (reinterpret_cast<uintptr_t>(a.output) & 15u) != 0)
        p.kind = ReducePlan::kFallback;
    uint64_t slices = p.slices;
    if (slices > 1) {
        const uint64_t fit = a.workspace == nullptr ? 0 : a.workspace_bytes / (p.pitch * sizeof(float));
        if (slices > fit) slices = fit > 1 ? fit : 1;
    }
    auto in = static_cast<const u32x4*>(a.input);
    switch (p.kind) {
        case ReducePlan::kRowsGrouped: {
            const uint64_t num_chunks = a.outer * p.chunks_per_row;
            constexpr int kU = 4;
            dim3 grid = blocks(num_chunks, kThreads * kU);
            switch (p.chunks_per_row) {
#define CQ_CASE(G) case G: hipLaunchKernelGGL((reduce_rows_grouped_kernel<F, G, kU>), grid, dim3(kThreads), 0, s, in, a.output, num_chunks); break;
                CQ_CASE(1) CQ_CASE(2) CQ_CASE(4) CQ_CASE(8) CQ_CASE(16) CQ_CASE(32) CQ_CASE(64)
#undef CQ_CASE
            }
            return hipGetLastError();
        }
        case ReducePlan::kRowsWave: {
            dim3 grid = blocks(a.outer * slices, kThreads / kWave);
            if (slices > 1) {
                hipLaunchKernelGGL((reduce_rows_wave_kernel<F, true>), grid, dim3(kThreads), 0, s, in, a.workspace, a.outer,
                                   p.chunks_per_row, static_cast<uint32_t>(slices), p.pitch);
                launch_fold<F>(s, a.workspace, a.output, slices, p.pitch, a.outer);
            } else {
                hipLaunchKernelGGL((reduce_rows_wave_kernel<F, false>), grid, dim3(kThreads), 0, s, in, a.output, a.outer,
                                   p.chunks_per_row, 1u, 0);
            }
            return hipGetLastError();
        }
        case ReducePlan::kCols: {
            dim3 grid = blocks(a.outer * p.inner_chunks * slices, kThreads);
            if (slices > 1) {
                hipLaunchKernelGGL((reduce_cols_kernel<F, true>), grid, dim3(kThreads), 0, s, in, a.workspace, a.outer, a.len,
                                   p.inner_chunks, static_cast<uint32_t>(slices));
                launch_fold<F>(s, a.workspace, a.output, slices, p.pitch, p.pitch);
            } else {
                hipLaunchKernelGGL((reduce_cols_kernel<F, false>), grid, dim3(kThreads), 0, s, in, a.output, a.outer, a.len,
                                   p.inner_chunks, 1u);
            }
            return hipGetLastError();
        }
        case ReducePlan::kTile: {
            const uint64_t jobs = a.outer * p.col_tiles * slices;
            if (slices > 1) {
                launch_tile<F, F, kThreads, kTilePartial>(s, p.cw, jobs, a.input, a.workspace, a.len, p.inner_chunks,
                                                          p.col_tiles, static_cast<uint32_t>(slices), p.pitch, 0);
                launch_fold<F>(s, a.workspace, a.output, slices, p.pitch, p.pitch);
            } else {
                launch_tile<F, F, kThreads, kTileFinalPacked>(s, p.cw, jobs, a.input, a.output, a.len, p.inner_chunks,
                                                              p.col_tiles, 1u, 0, 0);
            }
            return hipGetLastError();
        }
        case ReducePlan::kFallback: break;
    }
    StridedReduce r{};
    r.rank = a.rank;
    r.axis = a.axis;
    uint64_t num_out = 1;
    for (uint32_t d = 0; d < a.rank; d++) {
        r.shape[d] = static_cast<uint32_t>(a.shape[d]);
        r.in_strides[d] = a.in_strides[d];
        r.out_strides[d] = a.out_strides[d];
        if (d != a.axis) num_out *= a.shape[d];
    }
    if (num_out == 0) return hipSuccess;
    if (a.shape[a.axis] >= 256)
        hipLaunchKernelGGL((reduce_strided_kernel<F, kWave>), blocks(num_out * kWave, kThreads), dim3(kThreads), 0, s,
                           a.input, a.output, r, num_out);
    else
        hipLaunchKernelGGL((reduce_strided_kernel<F, 1>), blocks(num_out, kThreads), dim3(kThreads), 0, s, a.input,
                           a.output, r, num_out);
    return hipGetLastError();
}

}  // namespace

uint64_t reduce_workspace_bytes(uint64_t outer, uint64_t len, uint64_t inner, int dtype) {
    const ReducePlan p = plan_reduce(outer, len, inner, dtype == CQ_F32 ? 4 : 8);
    const uint64_t slices = p.slices > p.lane_slices ? p.slices : p.lane_slices;  // either kernel set may run
    // ... and room for the contiguous result of a launch whose output tensor turns out to be strided
    return (slices > 1 ? slices * p.pitch * sizeof(float) : 0) + packed_outputs_bytes(outer * inner, dtype == CQ_F32 ? 4 : 2);
}

hipError_t launch_reduce_max_abs(hipStream_t s, int dtype, const ReduceArgs& a) {
    switch (dtype) {
        case CQ_F32: return reduce_dispatch<F32>(s, a);
        case CQ_BF16: return reduce_dispatch<BF16>(s, a);
        case CQ_F16: return reduce_dispatch<F16>(s, a);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace cq
