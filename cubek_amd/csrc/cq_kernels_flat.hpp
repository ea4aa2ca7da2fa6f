// Kernel templates of the flat (contiguous) quantize / dequantize path for gfx950.
//
// Work decomposition.  The float tensor is cut into 16-byte chunks (8 bf16/f16
// or 4 f32 values).  Lane l of a kThreads-lane workgroup owns chunk
// (blockIdx*kUnroll + u)*kThreads + l for u = 0..kUnroll-1, so every
// global_load_dwordx4 / global_store_dwordx4 instruction of a wave covers one
// contiguous 1 KiB segment.  A quantization block of B elements spans
// kGroup = B / values-per-chunk adjacent lanes (a power of two inside one wave):
// its abs-max is a DPP butterfly, no LDS.  Codes narrower than a word
// (chunk bits 16 or 8) are OR-combined across 2 or 4 lanes before one store.
//
// quantize_flat_rows_kernel / dequantize_flat_rows_kernel run the same bodies over pitched rows: a
// row is a whole number of steps (kThreads chunks, the last one of a row may be partial), and a
// workgroup's kUnroll steps may lie in different rows.  quantize_flat_lanes_kernel /
// dequantize_flat_lanes_kernel do so for short rows and rows behind several levels of strides: there
// the lanes of one step lie in different rows and each finds its own.
//
// HBM traffic per element is the algorithmic minimum: the input once, the
// codes once, one scale per block.  Loads and stores carry the non-temporal
// hint: nothing is re-read.
#pragma once

#include "cq_device.hpp"
#include "cq_magic_div.hpp"

#ifndef CQ_WAVE_SCALES
#define CQ_WAVE_SCALES 1
#endif

namespace cq {

// Where a chunk's scale comes from.
enum ScaleSrc : int {
    kScaleDynamic = 0,     // abs-max of the block, computed here
    kScaleGivenF = 1,      // `scale_in`, typed like the input (the reference's `scale` argument)
    kScalePartials = 2,    // per tensor: `scale_in` holds the f32 abs-max partials of pass 1; this
                           // kernel (pass 2) finishes the reduction, derives the scale and quantizes
    kScaleStored = 3,      // `scale_in` holds the stored scales FS(F(scale)) of every block, written by an
                           // earlier launch and typed like the parameters: the divisor is F(stored), and
                           // nothing is written back (second pass of a two-launch dynamic quantize)
};

// ---- where the steps of a workgroup's tile lie -------------------------------------------------
// A tile is kUnroll steps of kThreads consecutive chunks, one per lane.  The kernel bodies ask a
// geometry, for each step u, for the (wave-uniform) base pointers of the tensors, the lane's chunk
// index relative to them (`chunk`; `load_chunk` is the same clamped into the data, for lanes past
// the end), whether the lane holds data (`live`), whether the step's row starts its blocks
// (`first_row`) and whether the lane holds the tensor's first chunk (`tensor_start`).  Scale i of a
// base pointer belongs to chunks [i * kDiv, (i + 1) * kDiv).

// One contiguous run of chunks [chunk_begin, chunk_end): the same pointers for every step.
template <int kUnroll, int kThreads, bool kChecked, bool kWaveRuns = false>
struct RunSteps;
struct RunGeo {
    const void* in;
    void* out;
    const void* scale_in;
    void* scale_out;
    uint64_t chunk_begin, chunk_end;
    static constexpr bool kWaveRuns = false;
    static constexpr bool kOneRun = true;  // every step reads the same tensors at consecutive chunks
    template <int kUnroll, int kThreads, bool kChecked>
    using Steps = RunSteps<kUnroll, kThreads, kChecked>;
};
// The same run with the tile's chunks dealt out wave by wave: a wave takes kUnroll * 64 consecutive chunks, step u
// of it the u-th 64 of them (RunGeo: step u of the workgroup is the u-th kThreads chunks of the tile).  Every load
// still covers 1 KiB; what changes is that the codes of a wave's steps lie next to each other, so that chunks of
// 8 or 16 bits of codes leave as one run of 256 or 512 bytes per wave instead of 64-byte pieces.
struct RunGeoWaves : RunGeo {
    static constexpr bool kWaveRuns = true;
    template <int kUnroll, int kThreads, bool kChecked>
    using Steps = RunSteps<kUnroll, kThreads, kChecked, true>;
};
template <int kUnroll, int kThreads, bool kChecked, bool kWaveRuns>
struct RunSteps {
    using Index = uint64_t;
    static constexpr int kStep = kWaveRuns ? kWave : kThreads;  // chunks from one step of a lane to its next
    const RunGeo& g;
    const uint64_t first;
    __device__ __forceinline__ RunSteps(const RunGeo& geo, uint32_t tile)
        : g(geo),
          first(geo.chunk_begin + static_cast<uint64_t>(tile) * (kThreads * kUnroll) +
                (kWaveRuns ? (threadIdx.x / kWave) * (kWave * kUnroll) + (threadIdx.x & (kWave - 1)) : threadIdx.x)) {}
    __device__ __forceinline__ Index chunk(int u) const { return first + static_cast<uint64_t>(u) * kStep; }
    // checked launches let out-of-range lanes re-read the last chunk instead of branching
    __device__ __forceinline__ Index load_chunk(int u) const {
        const Index c = chunk(u);
        return kChecked ? (c < g.chunk_end ? c : g.chunk_end - 1) : c;
    }
    __device__ __forceinline__ bool live(int u) const { return !kChecked || chunk(u) < g.chunk_end; }
    __device__ __forceinline__ bool first_row(int) const { return true; }
    __device__ __forceinline__ bool tensor_start(int u) const { return chunk(u) == 0; }
    __device__ __forceinline__ const void* in(int) const { return g.in; }
    __device__ __forceinline__ void* out(int) const { return g.out; }
    __device__ __forceinline__ const void* scale_in(int) const { return g.scale_in; }
    __device__ __forceinline__ void* scale_out(int) const { return g.scale_out; }
};

// Pitched rows.  A row of `row_chunks` chunks is `steps_per_row` steps, the last one partial where
// kThreads does not divide the row; step g of the launch is step g % steps_per_row of row
// g / steps_per_row.  The rows come in groups of `inner_rows`: the rows of a group start `in` / `out` /
// `scale_in` / `scale_out` bytes apart in the four tensors, the groups `*_outer` bytes (`*_wrap` =
// outer - inner_rows * inner, the step from a group's last row to the next group's first minus one row
// pitch).  Blocks of `scale_rows` rows (by a lane group of columns) share a row of scales (given scales
// only: a fused abs-max sees one row; one group of rows only).
struct FlatRows {
    uint32_t row_chunks, steps_per_row, total_steps;  // total_steps < 2^31
    uint32_t scale_rows;  // >= 1
    uint32_t inner_rows;
    // n / steps_per_row, n / inner_rows and n / scale_rows for n < 2^31 as (n * magic) >> shift (cq_magic_div.hpp)
    uint32_t steps_magic, steps_shift, inner_magic, inner_shift, scale_magic, scale_shift;
    uint64_t in, out, scale_in, scale_out;
    uint64_t in_outer, out_outer, scale_in_outer, scale_out_outer;
    uint64_t in_wrap, out_wrap, scale_in_wrap, scale_out_wrap;
};
template <int kUnroll, int kThreads, bool kChecked, int kInBytes, int kOutBytes, int kDiv>
struct RowSteps;
// kInBytes / kOutBytes: bytes of a chunk in `in` / `out`; kDiv: chunks per scale, 0 = one scale per tensor
template <int kInBytes, int kOutBytes, int kDiv>
struct RowsGeo {
    static constexpr bool kWaveRuns = false;
    static constexpr bool kOneRun = false;
    const void* in;
    void* out;
    const void* scale_in;
    void* scale_out;
    uint32_t step_begin;  // first step of the launch
    uint32_t scale_in_bytes, scale_out_bytes;  // bytes per scale
    FlatRows rows;
    template <int kUnroll, int kThreads, bool kChecked>
    using Steps = RowSteps<kUnroll, kThreads, kChecked, kInBytes, kOutBytes, kDiv>;
};
// The row and column of a step are wave-uniform, so each step's pointers are scalar arithmetic on
// the base pointers (the first step's by a multiplication, the following ones count on from it),
// and the lane's index is just its number in the workgroup.
template <int kUnroll, int kThreads, bool kChecked, int kInBytes, int kOutBytes, int kDiv>
struct RowSteps {
    using Index = uint32_t;
    const char* in_[kUnroll];
    char* out_[kUnroll];
    const char* scale_in_[kUnroll];
    char* scale_out_[kUnroll];
    uint32_t last_[kUnroll];  // last lane of the step that holds a chunk of its row
    bool valid_[kUnroll];     // the step exists (a checked launch may run past the last step)
    bool first_[kUnroll];
    __device__ __forceinline__ RowSteps(const RowsGeo<kInBytes, kOutBytes, kDiv>& g, uint32_t tile) {
        const FlatRows& r = g.rows;
        const uint32_t step = g.step_begin + tile * kUnroll;
        const uint32_t row = magic_div(step, r.steps_magic, r.steps_shift);
        uint32_t col = step - row * r.steps_per_row;
        const uint32_t group = magic_div(row, r.inner_magic, r.inner_shift);
        uint32_t lo = row - group * r.inner_rows;  // row within its group
        const uint32_t scale_row = magic_div(lo, r.scale_magic, r.scale_shift);
        uint32_t sub = lo - scale_row * r.scale_rows;
        bool first = kDiv == 0 ? step == 0 : sub == 0;
        // bytes from one step to the next one of the same row, and back to the row's first step
        constexpr uint64_t kScalesPerStep = kDiv == 0 ? 0 : kThreads / (kDiv == 0 ? 1 : kDiv);
        const uint64_t scale_in_step = kScalesPerStep * g.scale_in_bytes, scale_out_step = kScalesPerStep * g.scale_out_bytes;
        const uint64_t back = r.steps_per_row - 1;
        const char* in = static_cast<const char*>(g.in) + group * r.in_outer + lo * r.in +
                         static_cast<uint64_t>(col) * (kThreads * kInBytes);
        char* out = static_cast<char*>(g.out) + group * r.out_outer + lo * r.out +
                    static_cast<uint64_t>(col) * (kThreads * kOutBytes);
        const char* scale_in = static_cast<const char*>(g.scale_in) + group * r.scale_in_outer + scale_row * r.scale_in +
                               col * scale_in_step;
        char* scale_out = static_cast<char*>(g.scale_out) + group * r.scale_out_outer + scale_row * r.scale_out +
                          col * scale_out_step;
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            valid_[u] = !kChecked || u == 0 || step + u < r.total_steps;
            in_[u] = in;
            out_[u] = out;
            scale_in_[u] = scale_in;
            scale_out_[u] = g.scale_out == nullptr ? nullptr : scale_out;
            const uint32_t left = r.row_chunks - col * kThreads;
            last_[u] = left < kThreads ? left - 1 : kThreads - 1;
            first_[u] = first && valid_[u];
            // past the launch's last step the addresses stay where they are: on data
            if (kChecked && step + u + 1 >= r.total_steps) continue;
            if (++col != r.steps_per_row) {
                if (kDiv == 0) first = false;  // one scale per tensor: the launch's first step stores it
                in += kThreads * kInBytes;
                out += kThreads * kOutBytes;
                scale_in += scale_in_step;
                scale_out += scale_out_step;
            } else {  // on to the next row
                col = 0;
                in += r.in - back * (kThreads * kInBytes);
                out += r.out - back * (kThreads * kOutBytes);
                scale_in -= back * scale_in_step;
                scale_out -= back * scale_out_step;
                if (++sub == r.scale_rows) {
                    sub = 0;
                    scale_in += r.scale_in;
                    scale_out += r.scale_out;
                }
                if (++lo == r.inner_rows) {  // on to the next group of rows (scale_rows is 1 where there are several)
                    lo = 0;
                    in += r.in_wrap;
                    out += r.out_wrap;
                    scale_in += r.scale_in_wrap;
                    scale_out += r.scale_out_wrap;
                }
                first = kDiv == 0 ? false : sub == 0;
            }
        }
    }
    __device__ __forceinline__ Index chunk(int) const { return threadIdx.x; }
    __device__ __forceinline__ Index load_chunk(int u) const {
        return kChecked ? (threadIdx.x < last_[u] ? threadIdx.x : last_[u]) : threadIdx.x;
    }
    __device__ __forceinline__ bool live(int u) const { return !kChecked || (valid_[u] && threadIdx.x <= last_[u]); }
    __device__ __forceinline__ bool first_row(int u) const { return first_[u]; }
    __device__ __forceinline__ bool tensor_start(int u) const { return first_[u] && threadIdx.x == 0; }
    __device__ __forceinline__ const void* in(int u) const { return in_[u]; }
    __device__ __forceinline__ void* out(int u) const { return out_[u]; }
    __device__ __forceinline__ const void* scale_in(int u) const { return scale_in_[u]; }
    __device__ __forceinline__ void* scale_out(int u) const { return scale_out_[u]; }
};

// Short or irregularly strided rows (a head dimension behind permuted leading dimensions): the chunks
// of the launch are numbered through all rows, a step is kThreads consecutive ones, so the lanes of a
// step lie in several rows.  Each lane finds its row (chunk / row_chunks) and from it, dimension by
// dimension (innermost first, `count` entries each, multiply-and-shift divisions), the byte offsets of
// that row in the four tensors.  Blocks lie along the row, or (given scales) over rows of the innermost
// level as well, or there is one scale per tensor.
// kGroup of the lane-wise kernels that serve every block size: the lanes per block come with the launch
// (LaneRows::group_log2), one instantiation instead of one per block size.  Per tensor stays kGroup = 0.
constexpr int kGroupRt = -1;
constexpr int kParamRt = -1;  // the type of the stored scales is a launch argument
constexpr int kNearLaneLevels = kMaxLaneLevels;  // levels the lanes' short cut from their tile's first row walks (LaneRows::near)
struct LaneRows {
    uint32_t row_chunks, row_magic, row_shift;
    uint32_t total_chunks;  // < 2^31
    uint32_t levels;        // leading dimensions, 1 .. kMaxLaneLevels
    uint32_t narrow;        // every byte offset the rows can reach in the four tensors is below 2^32
    // narrow, no blocks over rows, at most kNearLaneLevels levels, and the innermost level is longer than the rows
    // one tile can span, its strides below 2^24 bytes: a tile's lanes find their rows from the tile's first row by
    // one step of at most one carry
    uint32_t near;
    // near, and rows of a power of two of chunks (1 + its log2 here; 0 = not so) that a step of the workgroup holds
    // whole, in a launch of whole tiles none of which runs over the end of the innermost level: a lane keeps its
    // column and its place among a step's rows for all of its chunks, and the step from chunk to chunk is the same
    // for every lane
    uint32_t whole_rows;
    uint32_t group_log2;    // lanes per block as a power of two, for the kernels that take it at run time (kGroupRt)
    // lanes per block where that is not a power of two (0: it is): blocks of 24 or 40 values ...  Only launches that
    // read their scales come with it (a fused abs-max needs the power of two for its butterfly): chunk / group_any
    // as a multiplication and a shift
    uint32_t group_any, group_magic, group_shift;
    // Tile order (0 = as numbered).  Where whole tiles fit the innermost level and the next level lies closer in
    // memory in the tensor that is read (heads next to each other behind positions, rows of 512 bytes and more),
    // workgroups that run together take the same tile of neighbouring entries of that level: slabs of order_inner x order_outer tiles are walked
    // outer entry first, and what the strided tensor sees are runs side by side instead of one run per workgroup.
    uint32_t order_inner, order_outer, order_outer_magic, order_outer_shift, order_slab_magic, order_slab_shift;
    // blocks of `scale_rows` entries of the innermost level (by a lane group of columns) share their scale
    // (given scales only); the scale strides of that level are per block of rows
    uint32_t scale_rows, scale_magic, scale_shift;
    uint32_t count[kMaxLaneLevels], magic[kMaxLaneLevels], shift[kMaxLaneLevels];
    uint64_t in[kMaxLaneLevels], out[kMaxLaneLevels], scale_in[kMaxLaneLevels], scale_out[kMaxLaneLevels];
};
template <int kUnroll, int kThreads>
struct LaneSteps;
struct LanesGeo {
    static constexpr bool kWaveRuns = false;
    static constexpr bool kOneRun = false;
    const void* in;
    void* out;
    const void* scale_in;
    void* scale_out;
    uint32_t tile_begin;  // first tile of the launch (a launch may cover the end of a numbering only)
    LaneRows rows;
    template <int kUnroll, int kThreads, bool kChecked>
    using Steps = LaneSteps<kUnroll, kThreads>;  // always checked
};
template <int kUnroll, int kThreads>
struct LaneSteps {
    using Index = uint32_t;
    const char* in_[kUnroll];
    char* out_[kUnroll];
    const char* scale_in_[kUnroll];
    char* scale_out_[kUnroll];
    uint32_t col_[kUnroll];  // the lane's chunk within its row
    bool live_[kUnroll], first_[kUnroll], block_row_[kUnroll];
    __device__ __forceinline__ LaneSteps(const LanesGeo& g, uint32_t tile_as_launched) {
        const LaneRows& r = g.rows;
        uint32_t tile = tile_as_launched;
        if (r.order_inner != 0) {  // only launches that start at tile 0 carry an order
            const uint32_t slab_tiles = r.order_inner * r.order_outer;
            const uint32_t slab = magic_div(tile, r.order_slab_magic, r.order_slab_shift);
            const uint32_t within = tile - slab * slab_tiles;
            const uint32_t inner = magic_div(within, r.order_outer_magic, r.order_outer_shift);
            const uint32_t outer = within - inner * r.order_outer;
            tile = slab * slab_tiles + outer * r.order_inner + inner;
        }
        // The shape of the launch is the same for every lane, so the cases below are scalar branches.
        if (r.levels == 1 && r.count[0] == 1) {
            // a single row (one contiguous run): chunk numbers are positions already
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                const uint32_t chunk = ((g.tile_begin + tile) * kUnroll + u) * kThreads + threadIdx.x;
                live_[u] = chunk < r.total_chunks;
                col_[u] = live_[u] ? chunk : r.total_chunks - 1;  // lanes past the end re-read the last chunk
                first_[u] = true;
                block_row_[u] = true;
                in_[u] = static_cast<const char*>(g.in);
                out_[u] = static_cast<char*>(g.out);
                scale_in_[u] = static_cast<const char*>(g.scale_in);
                scale_out_[u] = static_cast<char*>(g.scale_out);
            }
            return;
        }
        if (r.near) {
            // The tile's first row is the same for every lane: its digits and offsets come from the scalar unit.
            // A lane's row lies `drow` rows further on; when that runs over the end of the innermost level, the
            // carry walks up the levels that sit on their last entry, which the tile's first row decides too
            // (worked out only in the few tiles that hold such a lane).
            const uint32_t c0 = (g.tile_begin + tile) * (kUnroll * kThreads);  // < total_chunks
            const uint32_t row0 = magic_div(c0, r.row_magic, r.row_shift);
            const uint32_t col0 = c0 - row0 * r.row_chunks;
            uint32_t base[4] = {0, 0, 0, 0};  // narrow: every offset stays below 2^32
            uint32_t digits[kNearLaneLevels];
            uint32_t rest = row0;
#pragma unroll
            for (int l = 0; l < kNearLaneLevels; l++) {  // unrolled: the loads of every level's entries go out together
                digits[l] = 0;
                if (l < static_cast<int>(r.levels)) {
                    digits[l] = rest;
                    if (l + 1 < static_cast<int>(r.levels)) {
                        const uint32_t q = magic_div(rest, r.magic[l], r.shift[l]);
                        digits[l] = rest - q * r.count[l];
                        rest = q;
                    }
                    const uint32_t step[4] = {static_cast<uint32_t>(r.in[l]), static_cast<uint32_t>(r.out[l]),
                                              static_cast<uint32_t>(r.scale_in[l]), static_cast<uint32_t>(r.scale_out[l])};
#pragma unroll
                    for (int t = 0; t < 4; t++) base[t] += digits[l] * step[t];
                }
            }
            const uint32_t step0[4] = {static_cast<uint32_t>(r.in[0]), static_cast<uint32_t>(r.out[0]),
                                       static_cast<uint32_t>(r.scale_in[0]), static_cast<uint32_t>(r.scale_out[0])};
            if (r.whole_rows != 0) {
                const uint32_t log2 = r.whole_rows - 1;
                const uint32_t lane_row = threadIdx.x >> log2, col = threadIdx.x & (r.row_chunks - 1u);
                const uint32_t rows_per_step = kThreads >> log2;
                uint32_t off[4];
#pragma unroll
                for (int t = 0; t < 4; t++) off[t] = base[t] + __umul24(lane_row, step0[t]);
#pragma unroll
                for (int u = 0; u < kUnroll; u++) {
                    live_[u] = true;
                    col_[u] = col;
                    first_[u] = u == 0 && row0 == 0 && lane_row == 0;
                    block_row_[u] = true;
                    const uint32_t rows = u * rows_per_step;  // the same for every lane
                    in_[u] = static_cast<const char*>(g.in) + (off[0] + rows * step0[0]);
                    out_[u] = static_cast<char*>(g.out) + (off[1] + rows * step0[1]);
                    scale_in_[u] = static_cast<const char*>(g.scale_in) + (off[2] + rows * step0[2]);
                    scale_out_[u] = g.scale_out == nullptr ? nullptr : static_cast<char*>(g.scale_out) + (off[3] + rows * step0[3]);
                }
                return;
            }
            uint32_t drow[kUnroll];
            bool wraps[kUnroll], any_wraps = false;
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                const uint32_t chunk = c0 + u * kThreads + threadIdx.x;
                live_[u] = chunk < r.total_chunks;
                const uint32_t c = live_[u] ? chunk : r.total_chunks - 1;  // lanes past the end re-read the last chunk
                const uint32_t k = col0 + (c - c0);
                drow[u] = magic_div(k, r.row_magic, r.row_shift);
                col_[u] = k - __umul24(drow[u], r.row_chunks);
                first_[u] = row0 + drow[u] == 0;
                block_row_[u] = true;
                wraps[u] = digits[0] + drow[u] >= r.count[0];
                any_wraps = any_wraps || wraps[u];
            }
            uint32_t carried[4] = {0, 0, 0, 0};  // modulo 2^32: the sums it enters are exact
            if (__any(any_wraps)) {
                bool carry = true;
#pragma unroll
                for (int l = 0; l < kNearLaneLevels; l++) {
                    if (l < static_cast<int>(r.levels)) {
                        const uint32_t step[4] = {static_cast<uint32_t>(r.in[l]), static_cast<uint32_t>(r.out[l]),
                                              static_cast<uint32_t>(r.scale_in[l]), static_cast<uint32_t>(r.scale_out[l])};
                        const bool stays = l + 1 == static_cast<int>(r.levels) || digits[l] + 1 < r.count[l];  // a carry into this level ends here
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            if (l == 0)
                                carried[t] -= r.count[0] * step[t];
                            else if (carry)
                                carried[t] += stays ? step[t] : 0u - (r.count[l] - 1) * step[t];
                        }
                        if (l > 0 && stays) carry = false;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                uint32_t off[4];
#pragma unroll
                for (int t = 0; t < 4; t++) off[t] = base[t] + __umul24(drow[u], step0[t]) + (wraps[u] ? carried[t] : 0u);
                in_[u] = static_cast<const char*>(g.in) + off[0];
                out_[u] = static_cast<char*>(g.out) + off[1];
                scale_in_[u] = static_cast<const char*>(g.scale_in) + off[2];
                scale_out_[u] = g.scale_out == nullptr ? nullptr : static_cast<char*>(g.scale_out) + off[3];
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t chunk = ((g.tile_begin + tile) * kUnroll + u) * kThreads + threadIdx.x;
            live_[u] = chunk < r.total_chunks;
            const uint32_t c = live_[u] ? chunk : r.total_chunks - 1;  // lanes past the end re-read the last chunk
            uint32_t row = magic_div(c, r.row_magic, r.row_shift);
            col_[u] = c - row * r.row_chunks;
            first_[u] = row == 0;
            block_row_[u] = true;
            if (r.levels == 1 && r.narrow) {
                // rows in one uniform run (pitched rows, a slice) whose offsets fit 32 bits: no walk over levels
                uint32_t scale_row = row;
                if (r.scale_rows > 1) {
                    scale_row = magic_div(row, r.scale_magic, r.scale_shift);
                    block_row_[u] = row == scale_row * r.scale_rows;
                }
                in_[u] = static_cast<const char*>(g.in) + row * static_cast<uint32_t>(r.in[0]);
                out_[u] = static_cast<char*>(g.out) + row * static_cast<uint32_t>(r.out[0]);
                scale_in_[u] = static_cast<const char*>(g.scale_in) + scale_row * static_cast<uint32_t>(r.scale_in[0]);
                scale_out_[u] = g.scale_out == nullptr
                                    ? nullptr
                                    : static_cast<char*>(g.scale_out) + scale_row * static_cast<uint32_t>(r.scale_out[0]);
                continue;
            }
            uint64_t in = 0, out = 0, scale_in = 0, scale_out = 0;
#pragma unroll  // a loop over l would index the launch's arguments at run time, which sends all of them through scratch memory
            for (int l = 0; l < kMaxLaneLevels; l++) {
                if (l < static_cast<int>(r.levels)) {
                    uint32_t index = row;
                    if (l + 1 < static_cast<int>(r.levels)) {
                        const uint32_t q = magic_div(row, r.magic[l], r.shift[l]);
                        index = row - q * r.count[l];
                        row = q;
                    }
                    in += index * r.in[l];
                    out += index * r.out[l];
                    uint32_t scale_index = index;
                    if (l == 0 && r.scale_rows > 1) {
                        scale_index = magic_div(index, r.scale_magic, r.scale_shift);
                        block_row_[u] = index == scale_index * r.scale_rows;
                    }
                    scale_in += scale_index * r.scale_in[l];
                    scale_out += scale_index * r.scale_out[l];
                }
            }
            in_[u] = static_cast<const char*>(g.in) + in;
            out_[u] = static_cast<char*>(g.out) + out;
            scale_in_[u] = static_cast<const char*>(g.scale_in) + scale_in;
            scale_out_[u] = g.scale_out == nullptr ? nullptr : static_cast<char*>(g.scale_out) + scale_out;
        }
    }
    __device__ __forceinline__ Index chunk(int u) const { return col_[u]; }
    __device__ __forceinline__ Index load_chunk(int u) const { return col_[u]; }
    __device__ __forceinline__ bool live(int u) const { return live_[u]; }
    __device__ __forceinline__ bool first_row(int u) const { return block_row_[u]; }
    __device__ __forceinline__ bool tensor_start(int u) const { return first_[u] && col_[u] == 0; }
    __device__ __forceinline__ const void* in(int u) const { return in_[u]; }
    __device__ __forceinline__ void* out(int u) const { return out_[u]; }
    __device__ __forceinline__ const void* scale_in(int u) const { return scale_in_[u]; }
    __device__ __forceinline__ void* scale_out(int u) const { return scale_out_[u]; }
};

// kParam   : the type of the stored scales where the kernel is compiled for one (f32, or the float type of the
//            tensor itself); kParamRt: `param_dtype_rt` selects it at run time.
// kWide    : the value range does not fit its field (E4M3 / E5M2 in 8 bits).
// kChecked : the launch may run past `chunk_end` (ragged last tile): addresses
//            are clamped and stores masked.  Full tiles use the unchecked variant.
// kEnc     : stored encoding (kEncInt for the U32 store and native i8; e4m3 / e5m2 /
//            e2m1 for the native float stores, where kBits is the stored width).
template <class F, int kBits, int kGroup, int kScaleSrc, int kParam, bool kWide, int kUnroll,
          int kThreads, bool kChecked, int kEnc, class Geo>
__device__ __forceinline__ void quantize_flat_body(const Geo& geo, int param_dtype_rt, const QuantParams& qp,
                                                   uint32_t num_partials) {
    constexpr bool kDynamic = kScaleSrc == kScaleDynamic;
    static_assert(kScaleSrc != kScalePartials || kGroup == 0, "partials feed the per-tensor scale only");
    static_assert(kScaleSrc != kScaleStored || kGroup != 0, "stored scales are read back per block only");
    constexpr int kDiv = kGroup <= 0 ? 1 : kGroup;
    constexpr bool kRtGroup = kGroup == kGroupRt;
    uint32_t group_log2 = 0, group_any = 0, group_magic = 0, group_shift = 0;
    if constexpr (kRtGroup) {
        group_log2 = geo.rows.group_log2;
        if constexpr (!kDynamic) group_any = geo.rows.group_any, group_magic = geo.rows.group_magic, group_shift = geo.rows.group_shift;
    }
    // chunk -> its block, and whether it starts one (group_any is the same for the whole launch: scalar branches)
    const auto block_of = [&](auto c) {
        if constexpr (kRtGroup)
            return group_any != 0 ? static_cast<decltype(c)>(magic_div(static_cast<uint32_t>(c), group_magic, group_shift)) : c >> group_log2;
        else
            return c / kDiv;
    };
    const auto starts_block = [&](auto c) {
        if constexpr (kRtGroup)
            return group_any != 0 ? c == block_of(c) * group_any : (c & ((1u << group_log2) - 1u)) == 0;
        else
            return (c % kDiv) == 0;
    };
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;  // 64, 32, 16 or 8
    // chunks of less than a word of codes in a launch of whole tiles dealt out wave by wave: the words are stored
    // after the last step, one per lane
    constexpr bool kWordsLater = Geo::kWaveRuns && !kChecked && kChunkBits < 32 && kUnroll % (32 / (kChunkBits < 32 ? kChunkBits : 32)) == 0;
    [[maybe_unused]] uint32_t words[kUnroll];
    const int param_dtype = kParam != kParamRt ? kParam : param_dtype_rt;
    // Pass 2 of the per-tensor reduction walks the tiles last to first: pass 1 has just read the
    // tensor first to last, so what it read last is what the L2 caches still hold.  Groups of
    // eight consecutive tiles keep their places, because workgroup i runs on XCD i % 8 and tile
    // i was read there in pass 1 (each XCD has its own L2).
    uint32_t tile = blockIdx.x;
    if constexpr (kScaleSrc == kScalePartials) {
        const uint32_t whole = gridDim.x & ~7u;
        if (tile < whole) tile = (whole - 8 - (tile & ~7u)) + (tile & 7u);
    }
    const typename Geo::template Steps<kUnroll, kThreads, kChecked> at(geo, tile);

    // Given scales of a whole tile of one run: the 64 / kGroup scales a wave needs in each of its kUnroll steps come
    // with ONE load per lane (lane l fetches scale l % n of step l / n, n = 64 / kGroup) and reach their lanes through
    // ds_bpermute, instead of one load instruction per step in which kGroup lanes fetch the same scale (same-box A/B:
    // bf16 [14336, 4096] 4-bit 26.9 -> 26.2 us, f32 [8192, 8192] 2-bit 48.5 -> 46.8 us; dequantize of the former
    // 25.8 -> 25.2 us).
    constexpr bool kWaveScales = CQ_WAVE_SCALES && kScaleSrc == kScaleGivenF && Geo::kOneRun && !kChecked && kGroup >= 4 && kUnroll * (kWave / (kGroup > 0 ? kGroup : 1)) <= kWave;
    [[maybe_unused]] float s_wave = 0.0f;
    if constexpr (kWaveScales) {
        constexpr uint32_t kPerStep = kWave / kGroup;
        const uint32_t lane = threadIdx.x & (kWave - 1);
        const uint32_t su = lane / kPerStep, sj = lane % kPerStep;
        const auto c = (at.chunk(0) - lane) + su * (at.chunk(1) - at.chunk(0)) + sj * kGroup;
        if (su < kUnroll) s_wave = F::load_once(geo.scale_in, c / kGroup);
    }
    // All kUnroll loads are issued back to back.
    u32x4 raw[kUnroll];
    float s_given[kUnroll];
    RawScale s_stored[kUnroll];  // stored scales as loaded, widened behind the loads
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const auto c = at.load_chunk(u);
        raw[u] = stream_load(static_cast<const u32x4*>(at.in(u)) + c);
        if constexpr (kWaveScales)
            ;
        else if constexpr (kScaleSrc == kScaleStored)
            s_stored[u] = load_dtype_raw(param_dtype, at.scale_in(u), block_of(c));
        else if constexpr (!kDynamic && kGroup != 0 && kScaleSrc != kScalePartials)
            // read once, like the floats: with a plain load the launch takes 4 % longer where its codes are written
            // through the L2 (cfg5: 100.3 against 96.2 us).  Where the codes stream (outputs above 192 MiB) it is
            // the other way round by 3 % (8-bit codes of the same tensor: 115 against 112 us); choosing per launch
            // puts a branch among the loads, which costs the common case 1 - 5 %.
            s_given[u] = F::load_once(at.scale_in(u), block_of(c));
    }
    if constexpr (kScaleSrc == kScaleStored) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) s_given[u] = F::round(widen_dtype_raw(param_dtype, s_stored[u]));
    }
    if constexpr (kScaleSrc == kScalePartials) {
        // second pass of the grid reduction: every workgroup reduces the (<= a few
        // hundred) partial maxima again — max is exact, so all agree bit for bit
        const float* partials = static_cast<const float*>(geo.scale_in);
        float amax = 0.0f;
        for (uint32_t i = threadIdx.x; i < num_partials; i += kThreads) amax = fmaxf(amax, partials[i]);
        amax = group_max<64>(amax);
        __shared__ float wave_max[kThreads / kWave];
        if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = amax;
        __syncthreads();
        amax = wave_max[0];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; w++) amax = fmaxf(amax, wave_max[w]);
        const float s = F::round(scale_from_absmax(amax, qp.width));
#pragma unroll
        for (int u = 0; u < kUnroll; u++) s_given[u] = s;
    } else if constexpr (!kDynamic && kGroup == 0 && kScaleSrc != kScaleStored) {
        const float s = F::load(geo.scale_in, 0);  // one scale for the whole tensor
#pragma unroll
        for (int u = 0; u < kUnroll; u++) s_given[u] = s;
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic
    if constexpr (kWaveScales) {
        constexpr uint32_t kPerStep = kWave / kGroup;
        const uint32_t lane = threadIdx.x & (kWave - 1);
#pragma unroll
        for (int u = 0; u < kUnroll; u++)
            s_given[u] = bits_f32(static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>((u * kPerStep + lane / kGroup) * 4),
                                                                                      static_cast<int>(f32_bits(s_wave)))));
    }

#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const auto c = at.chunk(u);
        const bool live = at.live(u);
        uint32_t* const out = static_cast<uint32_t*>(at.out(u));
        void* const scale_out = at.scale_out(u);
        float v[kN];
        F::unpack(raw[u], v);

        float s_f;
        bool tame = false;
        if constexpr (kDynamic) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
            if constexpr (kRtGroup)
                amax = group_max_rt(amax, group_log2);
            else
                amax = group_max<kGroup>(amax);
            tame = absmax_is_tame(amax);
            const float s32 = tame ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
            s_f = F::round(s32);
        } else {
            s_f = s_given[u];
        }
        // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first lane.  s_f is an F value, so
        // FS rounds it only where FS is a 16-bit type other than F (the same for the whole launch: a scalar branch)
        const bool fs_rounds = param_dtype != CQ_F32 && param_dtype != F::kDtype;
        float s_fs = s_f;
        if (fs_rounds) s_fs = round_to_dtype(param_dtype, s_f);
        const auto si = kGroup == 0 ? 0 : block_of(c);
        const bool block_start = kGroup == 0 ? at.tensor_start(u) : (at.first_row(u) && starts_block(c));
        // (the scales leave through plain stores either way: written through like the codes below they cost 1 - 2 %)
        if constexpr (kScaleSrc != kScaleStored)
            if (scale_out != nullptr && live && block_start) store_dtype(param_dtype, scale_out, si, s_fs);
        // divisor F(FS(scale)): s_f itself unless FS rounded it
        float d = s_f;
        if (fs_rounds) d = F::round(s_fs);
        if constexpr (kScaleSrc == kScaleStored) d = s_f;  // F(stored) as loaded
        // a tame abs-max gives a tame scale; every other divisor is looked at itself
        if (!(kDynamic && F::kDtype != CQ_F16) || fs_rounds) tame = divisor_is_tame(d);

        uint32_t w[2];
        const auto by_value = [&](bool d_tame) {
            float qn[kN];  // negated codes
            quantize_codes<F, kN, kEnc>(v, d, d_tame, qp.lo, qp.hi, qp.unrounded != 0, qn);
            if constexpr (kEnc == kEncInt)
                pack_chunk_neg<kBits, kN, kWide>(qn, w);
            else
                encode_chunk<kEnc, kN>(qn, w);
        };
        if constexpr (F::kDtype == CQ_F16 && kEnc == kEncInt && !kWide) {
            if (tame)
                quantize_pack_f16_tame<kBits>(v, d, qp.lo, qp.hi, w);
            else
                by_value(false);
        } else {
            by_value(tame);
        }

        const bool keep = qp.keep != 0;
        if constexpr (kChunkBits == 64) {
            if (live) output_store(keep, u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(out) + c);
        } else if constexpr (kChunkBits == 32) {
            if (live) output_store(keep, w[0], out + c);
        } else {
            constexpr int kLanesPerWord = 32 / kChunkBits;  // 2 or 4
            const uint32_t sub = static_cast<uint32_t>(c) & (kLanesPerWord - 1);
            const uint32_t word = group_or<kLanesPerWord>(w[0] << (sub * kChunkBits));
            if constexpr (kWordsLater)
                words[u] = word;  // every lane of the word holds it: stored below
            else if (live && sub == 0)
                output_store(keep, word, out + c / kLanesPerWord);
        }
    }
    if constexpr (kWordsLater) {
        // A wave's steps are neighbours in memory (RunGeoWaves): lane `sub` of a word's lanes stores the word of
        // step g * kLanesPerWord + sub, so every lane stores and a wave's store covers kLanesPerWord * 64 bytes in a row.
        constexpr int kLanesPerWord = 32 / kChunkBits;
        const bool keep = qp.keep != 0;
        const uint32_t sub = threadIdx.x & (kLanesPerWord - 1);
#pragma unroll
        for (int g = 0; g < kUnroll / kLanesPerWord; g++) {
            uint32_t mine = words[g * kLanesPerWord];
#pragma unroll
            for (int j = 1; j < kLanesPerWord; j++) mine = sub == static_cast<uint32_t>(j) ? words[g * kLanesPerWord + j] : mine;
            const auto c = at.chunk(g * kLanesPerWord) + sub * (kWave);
            output_store(keep, mine, static_cast<uint32_t*>(at.out(0)) + c / kLanesPerWord);
        }
    }
}

// One contiguous run of whole tiles, parameters typed f32 or like the tensor (kParam): the hot launch.  Ragged
// ends, other parameter types and rows that are not whole steps run lane by lane (quantize_flat_lanes_kernel),
// which keeps the number of kernels in the library, and with it its size and load time, down.
template <class F, int kBits, int kGroup, int kScaleSrc, bool kWide, int kUnroll, int kThreads, int kEnc = kEncInt,
          int kParam = CQ_F32>
__global__ __launch_bounds__(kThreads) void quantize_flat_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, uint64_t chunk_begin, uint64_t chunk_end, QuantParams qp, uint32_t num_partials) {
    const RunGeo geo{in, out, scale_in, scale_out, chunk_begin, chunk_end};
    if constexpr (F::kPerChunk * kBits < 32) {  // less than a word of codes per chunk
        const RunGeoWaves waves{geo};
        quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParam, kWide, kUnroll, kThreads, false, kEnc>(waves, kParam, qp, num_partials);
    } else {
        quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParam, kWide, kUnroll, kThreads, false, kEnc>(geo, kParam, qp, num_partials);
    }
}

// Pitched rows of whole steps, from step `step_begin` of the launch on, parameters as in quantize_flat_kernel.  A kernel of its own
// so that the launches over one contiguous run carry none of the row arithmetic in their prologue.
template <class F, int kBits, int kGroup, int kScaleSrc, bool kWide, int kUnroll, int kThreads, int kEnc = kEncInt,
          int kParam = CQ_F32>
__global__ __launch_bounds__(kThreads) void quantize_flat_rows_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, uint32_t step_begin, QuantParams qp, uint32_t num_partials, FlatRows rows) {
    const RowsGeo<16, F::kPerChunk * kBits / 8, kGroup> geo{in, out, scale_in, scale_out, step_begin, F::kBytes,
                                                            kParam == CQ_F32 ? 4 : 2, rows};
    quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParam, kWide, kUnroll, kThreads, false, kEnc>(geo, kParam, qp, num_partials);
}

// Rows found lane by lane (LaneSteps), bounds-checked; the scale type is read at run time.  `tile_begin`:
// the launch starts at that tile of the numbering (the ragged end behind a launch of whole tiles).
template <class F, int kBits, int kGroup, int kScaleSrc, bool kWide, int kUnroll, int kThreads, int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void quantize_flat_lanes_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, int param_dtype_rt, QuantParams qp, uint32_t num_partials, uint32_t tile_begin,
    LaneRows rows) {
    const LanesGeo geo{in, out, scale_in, scale_out, tile_begin, rows};
    quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParamRt, kWide, kUnroll, kThreads, true, kEnc>(geo, param_dtype_rt, qp,
                                                                                               num_partials);
}

// `scale_in` of the geometry holds the stored scales
template <class F, int kBits, int kGroup, int kParam, int kUnroll, int kThreads, bool kChecked, int kEnc, class Geo>
__device__ __forceinline__ void dequantize_flat_body(const Geo& geo, int param_dtype_rt) {
    const int param_dtype = kParam != kParamRt ? kParam : param_dtype_rt;
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    const typename Geo::template Steps<kUnroll, kThreads, kChecked> at(geo, blockIdx.x);

    // the scales of a wave's kUnroll steps through one load per lane and ds_bpermute (see quantize_flat_body); 16-bit
    // outputs only (f32 [8192, 8192], 2-bit codes on blocks of 64: 45.4 us with it, 44.6 us without)
    constexpr bool kWaveScales = CQ_WAVE_SCALES && kParam == CQ_F32 && F::kBytes == 2 && Geo::kOneRun && !kChecked && kGroup >= 4 && kUnroll * (kWave / (kGroup > 0 ? kGroup : 1)) <= kWave;
    [[maybe_unused]] float sc_wave = 0.0f;
    if constexpr (kWaveScales) {
        constexpr uint32_t kPerStep = kWave / kGroup;
        const uint32_t lane = threadIdx.x & (kWave - 1);
        const uint32_t su = lane / kPerStep, sj = lane % kPerStep;
        const auto c = (at.chunk(0) - lane) + su * (kUnroll > 1 ? at.chunk(kUnroll > 1 ? 1 : 0) - at.chunk(0) : 0) + sj * kGroup;
        if (su < kUnroll) sc_wave = F32::load(geo.scale_in, c / kGroup);
    }
    uint32_t w0[kUnroll], w1[kUnroll];
    RawScale sc_raw[kUnroll];  // scales as loaded: nothing in the loop below waits for a load
    float sc[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const auto c = at.load_chunk(u);
        const uint32_t* const in = static_cast<const uint32_t*>(at.in(u));
        w1[u] = 0;
        if constexpr (kChunkBits == 64) {
            u32x2 w = stream_load(reinterpret_cast<const u32x2*>(in) + c);
            w0[u] = w[0];
            w1[u] = w[1];
        } else if constexpr (kChunkBits == 32) {
            w0[u] = stream_load(in + c);
        } else {
            constexpr int kLanesPerWord = 32 / kChunkBits;
            uint32_t w = in[c / kLanesPerWord];  // neighbouring lanes share the word
            w0[u] = w >> ((static_cast<uint32_t>(c) & (kLanesPerWord - 1)) * kChunkBits);
        }
        auto si = kGroup == 0 ? 0 : c / (kGroup <= 0 ? 1 : kGroup);
        if constexpr (kGroup == kGroupRt)
            si = geo.rows.group_any != 0 ? magic_div(c, geo.rows.group_magic, geo.rows.group_shift) : c >> geo.rows.group_log2;
        if constexpr (kWaveScales)
            ;
        else if constexpr (kParam == CQ_F32)
            sc[u] = F32::load(at.scale_in(u), si);  // a plain load: streamed, the launch takes 4 % longer
        else
            sc_raw[u] = load_dtype_raw(param_dtype, at.scale_in(u), si);
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic
    if constexpr (kWaveScales) {
        constexpr uint32_t kPerStep = kWave / kGroup;
        const uint32_t lane = threadIdx.x & (kWave - 1);
#pragma unroll
        for (int u = 0; u < kUnroll; u++)
            sc[u] = bits_f32(static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>((u * kPerStep + lane / kGroup) * 4),
                                                                                 static_cast<int>(f32_bits(sc_wave)))));
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++)  // Line::cast_from(scale)
        sc[u] = F::round(kParam == CQ_F32 ? sc[u] : widen_dtype_raw(param_dtype, sc_raw[u]));
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        float y[kN];
        if constexpr (kChunkBits == 64) {
            decode_fields<kEnc, kBits, 4>(w0[u], y);
            decode_fields<kEnc, kBits, 4>(w1[u], y + 4);
        } else {
            decode_fields<kEnc, kBits, kN>(w0[u], y);
        }
#pragma unroll
        for (int i = 0; i < kN; i++) y[i] = sc[u] * y[i];
        if (at.live(u)) stream_store(F::pack(y), static_cast<u32x4*>(at.out(u)) + at.chunk(u));  // pack rounds to F
    }
}

// whole tiles of one contiguous run, parameters typed f32 or like the tensor (see quantize_flat_kernel)
template <class F, int kBits, int kGroup, int kUnroll, int kThreads, int kEnc = kEncInt, int kParam = CQ_F32>
__global__ __launch_bounds__(kThreads) void dequantize_flat_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params, uint64_t chunk_begin,
    uint64_t chunk_end) {
    const RunGeo geo{in, out, params, nullptr, chunk_begin, chunk_end};
    dequantize_flat_body<F, kBits, kGroup, kParam, kUnroll, kThreads, false, kEnc>(geo, kParam);
}
// pitched rows of whole steps
template <class F, int kBits, int kGroup, int kUnroll, int kThreads, int kEnc = kEncInt, int kParam = CQ_F32>
__global__ __launch_bounds__(kThreads) void dequantize_flat_rows_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params, uint32_t step_begin,
    FlatRows rows) {
    const RowsGeo<F::kPerChunk * kBits / 8, 16, kGroup> geo{in, out, params, nullptr, step_begin, kParam == CQ_F32 ? 4 : 2, 0, rows};
    dequantize_flat_body<F, kBits, kGroup, kParam, kUnroll, kThreads, false, kEnc>(geo, kParam);
}
// lane by lane, bounds-checked, parameter type read at run time
template <class F, int kBits, int kGroup, int kUnroll, int kThreads, int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void dequantize_flat_lanes_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params, int param_dtype_rt,
    uint32_t tile_begin, LaneRows rows) {
    const LanesGeo geo{in, out, params, nullptr, tile_begin, rows};
    dequantize_flat_body<F, kBits, kGroup, kParamRt, kUnroll, kThreads, true, kEnc>(geo, param_dtype_rt);
}

// Block abs-max -> scale typed like the input (what quantize takes as `scale`).
template <class F, int kGroup, int kUnroll, int kThreads, class Geo>
__device__ __forceinline__ void scales_flat_body(const Geo& geo, const QuantParams& qp) {
    constexpr int kN = F::kPerChunk;
    const typename Geo::template Steps<kUnroll, kThreads, true> at(geo, blockIdx.x);
    u32x4 raw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) raw[u] = stream_load(static_cast<const u32x4*>(at.in(u)) + at.load_chunk(u));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const auto c = at.chunk(u);
        float v[kN];
        F::unpack(raw[u], v);
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
        bool starts;
        auto block = c;
        if constexpr (kGroup == kGroupRt) {
            const uint32_t log2 = geo.rows.group_log2;
            amax = group_max_rt(amax, log2);
            starts = (c & ((1u << log2) - 1u)) == 0;
            block = c >> log2;
        } else {
            amax = group_max<kGroup>(amax);
            starts = (c % kGroup) == 0;
            block = c / kGroup;
        }
        const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp)
                                               : scale_from_absmax(amax, qp.width);
        if (at.live(u) && starts) F::store(at.scale_out(u), block, s32);
    }
}

template <class F, int kGroup, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void scales_flat_kernel(const u32x4* __restrict__ in,
                                                               void* __restrict__ scales,
                                                               uint64_t num_chunks, QuantParams qp) {
    const RunGeo geo{in, nullptr, nullptr, scales, 0, num_chunks};
    scales_flat_body<F, kGroup, kUnroll, kThreads>(geo, qp);
}
// pitched rows: rows.in / rows.scale_out bytes between the rows of the two tensors
template <class F, int kGroup, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void scales_flat_rows_kernel(const u32x4* __restrict__ in,
                                                                    void* __restrict__ scales, QuantParams qp,
                                                                    FlatRows rows) {
    const RowsGeo<16, 0, kGroup> geo{in, nullptr, nullptr, scales, 0, 0, F::kBytes, rows};
    scales_flat_body<F, kGroup, kUnroll, kThreads>(geo, qp);
}

template <class F, int kGroup, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void scales_flat_lanes_kernel(const u32x4* __restrict__ in,
                                                                     void* __restrict__ scales, QuantParams qp,
                                                                     LaneRows rows) {
    const LanesGeo geo{in, nullptr, nullptr, scales, 0, rows};
    scales_flat_body<F, kGroup, kUnroll, kThreads>(geo, qp);
}

// Per-tensor abs-max, pass 1: grid-stride over chunks with kUnroll 16-byte loads
// in flight per lane, one partial per workgroup.  Lanes past the end re-read the
// last chunk (harmless for a maximum).  kAligned = false: element-wise loads for
// tensors that do not start on a 16-byte boundary.
template <class F, int kThreads, int kUnroll, bool kAligned>
__global__ __launch_bounds__(kThreads) void absmax_partials_kernel(const void* __restrict__ input,
                                                                   uint64_t num_elems,
                                                                   float* __restrict__ partials) {
    constexpr int kN = F::kPerChunk;
    const uint64_t gid = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const uint64_t total = static_cast<uint64_t>(gridDim.x) * kThreads;
    float amax = 0.0f;
    if constexpr (kAligned) {
        const u32x4* in = static_cast<const u32x4*>(input);
        const uint64_t num_chunks = num_elems / kN;
        if (num_chunks > 0) {
            for (uint64_t c0 = gid; c0 < num_chunks; c0 += total * kUnroll) {
                u32x4 raw[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; u++) {
                    const uint64_t c = c0 + static_cast<uint64_t>(u) * total;
                    // a plain load, not a streaming one: pass 2 reads the tensor again, and what stays in the L2
                    // and the Infinity Cache from here it does not fetch from HBM (tensors of 32 MiB: 16.4 -> 13.0 us
                    // for both passes, 128 MiB: 54.6 -> 50.5 us, 448 MiB: 181 -> 177 us)
                    raw[u] = in[c < num_chunks ? c : num_chunks - 1];
                }
#pragma unroll
                for (int u = 0; u < kUnroll; u++) {
                    float v[kN];
                    F::unpack(raw[u], v);
#pragma unroll
                    for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
                }
            }
        }
        if (gid == 0) {  // ragged tail, fewer than one chunk
            for (uint64_t e = num_chunks * kN; e < num_elems; e++) amax = fmaxf(amax, fabsf(F::load(input, e)));
        }
    } else {
        for (uint64_t e = gid; e < num_elems; e += total) amax = fmaxf(amax, fabsf(F::load(input, e)));
    }
    amax = group_max<64>(amax);
    __shared__ float wave_max[kThreads / kWave];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = wave_max[0];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; w++) m = fmaxf(m, wave_max[w]);
        partials[blockIdx.x] = m;
    }
}

// Per-tensor scale from the partials: value = via(F(2*absmax/width)) stored as `out_dtype`.
template <int kThreads>
__global__ __launch_bounds__(kThreads) void tensor_scale_kernel(const float* __restrict__ partials,
                                                                uint32_t num_partials, float width,
                                                                int f_dtype, int out_dtype,
                                                                void* __restrict__ out) {
    float amax = 0.0f;
    for (uint32_t i = threadIdx.x; i < num_partials; i += kThreads) amax = fmaxf(amax, partials[i]);
    amax = group_max<64>(amax);
    __shared__ float wave_max[kThreads / kWave];
    if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = wave_max[0];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; w++) m = fmaxf(m, wave_max[w]);
        float s_f = round_to_dtype(f_dtype, scale_from_absmax(m, width));
        store_dtype(out_dtype, out, 0, round_to_dtype(out_dtype, s_f));
    }
}

}  // namespace cq
