// Shared by the translation units that launch the flat kernels (cq_kernels_flat*.hip): launch
// shapes, tile splitting, the dispatch macros, and the quantize launch chain, which each unit
// instantiates for its own scale sources.
#pragma once

#include <type_traits>
#include "cq_internal.hpp"
#include "cq_kernels_flat.hpp"

namespace cq {

// The quantize launchers, one per float type, family of scale sources (0: produced in the launch, 1: given) and
// width of the codes, each compiled from cq_kernels_flat_quantize.hip into an object of its own: the runtime loads
// an object's code on the first launch out of it, and what a process's first quantize call waits for is the size of
// that one object.
#define CQ_QUANTIZE_FLAT_TU_(f, g, b) launch_quantize_flat_##f##_##g##_##b
#define CQ_QUANTIZE_FLAT_TU(f, g, b) CQ_QUANTIZE_FLAT_TU_(f, g, b)
#define CQ_DECLARE_QUANTIZE_TU(f, g)                                                             \
    hipError_t CQ_QUANTIZE_FLAT_TU(f, g, 2)(hipStream_t s, ScaleSource src, const FlatArgs& a); \
    hipError_t CQ_QUANTIZE_FLAT_TU(f, g, 4)(hipStream_t s, ScaleSource src, const FlatArgs& a); \
    hipError_t CQ_QUANTIZE_FLAT_TU(f, g, 8)(hipStream_t s, ScaleSource src, const FlatArgs& a);
CQ_DECLARE_QUANTIZE_TU(F32, 0)
CQ_DECLARE_QUANTIZE_TU(F32, 1)
CQ_DECLARE_QUANTIZE_TU(BF16, 0)
CQ_DECLARE_QUANTIZE_TU(BF16, 1)
CQ_DECLARE_QUANTIZE_TU(F16, 0)
CQ_DECLARE_QUANTIZE_TU(F16, 1)
#undef CQ_DECLARE_QUANTIZE_TU
// The whole-tile kernels of a contiguous run for parameters typed like the float tensor (bf16 scales of a bf16
// tensor, f16 of f16) live in objects of their own (-DCQ_TU_SAME=1): the runtime loads an object's code on its
// first launch, so launches with f32 parameters do not pay for them.  FlatArgs::whole_grid tiles, nothing else.
#ifndef CQ_TU_SAME
#define CQ_TU_SAME 0
#endif
#define CQ_QUANTIZE_FLAT_SAME_TU_(f, g) launch_quantize_flat_same_##f##_##g
#define CQ_QUANTIZE_FLAT_SAME_TU(f, g) CQ_QUANTIZE_FLAT_SAME_TU_(f, g)
hipError_t CQ_QUANTIZE_FLAT_SAME_TU(BF16, 0)(hipStream_t s, int bits, ScaleSource src, const FlatArgs& a);
hipError_t CQ_QUANTIZE_FLAT_SAME_TU(BF16, 1)(hipStream_t s, int bits, ScaleSource src, const FlatArgs& a);
hipError_t CQ_QUANTIZE_FLAT_SAME_TU(F16, 0)(hipStream_t s, int bits, ScaleSource src, const FlatArgs& a);
hipError_t CQ_QUANTIZE_FLAT_SAME_TU(F16, 1)(hipStream_t s, int bits, ScaleSource src, const FlatArgs& a);
#define CQ_DEQUANTIZE_FLAT_SAME_TU_(f) launch_dequantize_flat_same_##f
#define CQ_DEQUANTIZE_FLAT_SAME_TU(f) CQ_DEQUANTIZE_FLAT_SAME_TU_(f)
hipError_t CQ_DEQUANTIZE_FLAT_SAME_TU(BF16)(hipStream_t s, int bits, const FlatArgs& a);
hipError_t CQ_DEQUANTIZE_FLAT_SAME_TU(F16)(hipStream_t s, int bits, const FlatArgs& a);
template <class F>
hipError_t quantize_flat_same(bool given, hipStream_t s, int bits, ScaleSource src, const FlatArgs& a) {
    if constexpr (std::is_same_v<F, BF16>)
        return given ? CQ_QUANTIZE_FLAT_SAME_TU(BF16, 1)(s, bits, src, a) : CQ_QUANTIZE_FLAT_SAME_TU(BF16, 0)(s, bits, src, a);
    else if constexpr (std::is_same_v<F, F16>)
        return given ? CQ_QUANTIZE_FLAT_SAME_TU(F16, 1)(s, bits, src, a) : CQ_QUANTIZE_FLAT_SAME_TU(F16, 0)(s, bits, src, a);
    else
        return hipErrorInvalidValue;
}
template <class F>
hipError_t dequantize_flat_same(hipStream_t s, int bits, const FlatArgs& a) {
    if constexpr (std::is_same_v<F, BF16>)
        return CQ_DEQUANTIZE_FLAT_SAME_TU(BF16)(s, bits, a);
    else if constexpr (std::is_same_v<F, F16>)
        return CQ_DEQUANTIZE_FLAT_SAME_TU(F16)(s, bits, a);
    else
        return hipErrorInvalidValue;
}

// the dequantize launchers, one per float type and width of the codes (cq_kernels_flat_dequantize.hip)
#define CQ_DEQUANTIZE_FLAT_TU_(f, b) launch_dequantize_flat_##f##_##b
#define CQ_DEQUANTIZE_FLAT_TU(f, b) CQ_DEQUANTIZE_FLAT_TU_(f, b)
#define CQ_DECLARE_DEQUANTIZE_TU(f)                                            \
    hipError_t CQ_DEQUANTIZE_FLAT_TU(f, 2)(hipStream_t s, const FlatArgs& a); \
    hipError_t CQ_DEQUANTIZE_FLAT_TU(f, 4)(hipStream_t s, const FlatArgs& a); \
    hipError_t CQ_DEQUANTIZE_FLAT_TU(f, 8)(hipStream_t s, const FlatArgs& a);
CQ_DECLARE_DEQUANTIZE_TU(F32)
CQ_DECLARE_DEQUANTIZE_TU(BF16)
CQ_DECLARE_DEQUANTIZE_TU(F16)
#undef CQ_DECLARE_DEQUANTIZE_TU

namespace {

constexpr int kThreads = 256;

inline uint32_t grid_for(uint64_t num_chunks, int unroll) {
    uint64_t per = static_cast<uint64_t>(kThreads) * unroll;
    return static_cast<uint32_t>((num_chunks + per - 1) / per);
}

int group_of(int dtype, uint32_t block) {
    if (block == 0) return 0;
    uint32_t per_chunk = dtype == CQ_F32 ? 4u : 8u;
    if (block % per_chunk) return -1;
    uint32_t g = block / per_chunk;
    if (g & (g - 1)) return -1;
    return g <= 32 ? static_cast<int>(g) : -1;
}

// two's-complement fields of a value range wider than 8 bits (E4M3 / E5M2 in the U32 store)
inline bool fields_wrap(const FlatArgs& a) { return a.encoding == 0 && (a.range.hi > 127.0f || a.range.lo < -128.0f); }

// Chunks per block of a block size that group_of() refuses although it is a whole number of chunks (not a power of
// two, or more than 32): the lane-wise kernels divide by it, for launches that read their scales.  0: none.
uint32_t any_group_of(int dtype, uint32_t block) {
    const uint32_t per_chunk = dtype == CQ_F32 ? 4u : 8u;
    if (block == 0 || block % per_chunk != 0 || group_of(dtype, block) >= 0) return 0;
    return block / per_chunk;
}
// the power-of-two group whose launch shape (loads in flight) a launch with any_group_of() chunks per block takes
inline int shape_group_of(uint32_t any_group) { return any_group <= 8 ? 8 : 16; }

// Which lane groups (16-byte chunks per block) have kernels over whole tiles of a contiguous run, and over whole
// steps of pitched rows: one scale per tensor and blocks of 4 to 32 (4 to 16) chunks, i.e. 32 - 256 values of a 16-bit
// type, 16 - 128 of f32.  Blocks of one or two chunks run lane by lane: a kernel per block size, float type, code
// width and scale source is what makes the library large and its first launch slow.
constexpr bool whole_tiles_for(int group) { return group == 0 || group >= 4; }
constexpr bool whole_steps_for(int group) { return group == 0 || (group >= 4 && group <= 16); }

// Launch shapes from a sweep on MI355X (batches of back-to-back launches,
// 117 MB - 470 MB tensors): quantize is best with four 16-byte loads in flight
// per lane; dequantize, which is store-dominated, with two 16-byte stores per lane
// for 16-bit outputs.  For f32 outputs the best depth follows the share of reads:
// four stores per lane where the codes and scales are under ~15 % of the bytes
// written (measured 87-91 % of HBM peak against 78-87 % with two), two stores
// where they are more (8-bit codes, 4-bit codes with blocks of 32: 81-83 % against 73-75 %).
constexpr int kUnrollQ = 4;
template <class F, int kBits, int kGroup>
constexpr int kUnrollD = F::kBytes != 4 ? 2 : ((kBits == 8 || (kBits == 4 && kGroup > 0 && kGroup <= 8)) ? 2 : 4);

// the rows of a launch as the kernels take them: steps of kThreads chunks, a row's last one partial
FlatRows flat_rows(const FlatArgs& a) {
    FlatRows r;
    r.row_chunks = static_cast<uint32_t>(a.num_chunks);
    r.steps_per_row = static_cast<uint32_t>((a.num_chunks + kThreads - 1) / kThreads);
    r.total_steps = static_cast<uint32_t>(a.rows * r.steps_per_row);
    r.scale_rows = a.scale_rows > 1 ? a.scale_rows : 1u;
    r.inner_rows = static_cast<uint32_t>(a.inner_rows == 0 ? a.rows : a.inner_rows);
    magic_of(r.steps_per_row, &r.steps_magic, &r.steps_shift);
    magic_of(r.inner_rows, &r.inner_magic, &r.inner_shift);
    magic_of(r.scale_rows, &r.scale_magic, &r.scale_shift);
    r.in = a.in_pitch;
    r.out = a.out_pitch;
    r.scale_in = a.scale_in_pitch;
    r.scale_out = a.scale_out_pitch;
    r.in_outer = a.in_outer;
    r.out_outer = a.out_outer;
    r.scale_in_outer = a.scale_in_outer;
    r.scale_out_outer = a.scale_out_outer;
    // unsigned wrap-around is meant: an outer pitch may be smaller than a group of rows (permuted dimensions)
    r.in_wrap = a.in_outer - r.inner_rows * a.in_pitch;
    r.out_wrap = a.out_outer - r.inner_rows * a.out_pitch;
    r.scale_in_wrap = a.scale_in_outer - r.inner_rows * a.scale_in_pitch;
    r.scale_out_wrap = a.scale_out_outer - r.inner_rows * a.scale_out_pitch;
    return r;
}

// The lane-wise kernels take the lanes per block at run time (one instantiation for every block size); one scale
// per tensor (kGroup 0) stays a kernel of its own.
constexpr int lanes_group(int group) { return group == 0 ? 0 : kGroupRt; }
inline LaneRows with_group(LaneRows r, int group, uint32_t any_group = 0) {
    r.group_log2 = 0;
    while ((1 << r.group_log2) < group) r.group_log2++;
    r.group_any = any_group;
    if (any_group != 0) magic_of(any_group, &r.group_magic, &r.group_shift);
    return r;
}
// the most chunks a tile of the lane-wise kernels holds (threads x the deepest unroll in use)
constexpr uint32_t kLaneTileChunks = kThreads * 8;
// Whether every byte offset the rows of `r` can reach stays below 2^32 in each of the four tensors.
void set_narrow(LaneRows* r) {
    uint64_t reach[4] = {0, 0, 0, 0};
    for (uint32_t l = 0; l < r->levels; l++) {
        const uint64_t last = r->count[l] - 1;
        const uint64_t steps[4] = {r->in[l], r->out[l], r->scale_in[l], r->scale_out[l]};
        for (int t = 0; t < 4; t++) {
            if (last != 0 && steps[t] > (1ull << 32) / last) {
                r->narrow = 0;
                return;
            }
            reach[t] += last * steps[t];
        }
    }
    r->narrow = 1;
    for (int t = 0; t < 4; t++)
        if (reach[t] >= (1ull << 32)) r->narrow = 0;
}
// Whether the lanes of a tile can find their rows from the tile's first row (LaneRows::near): the rows one tile
// spans (at most kLaneTileChunks chunks) run over the end of the innermost level once at most.
void set_near(LaneRows* r) {
    const uint64_t span = kLaneTileChunks / r->row_chunks + 2;
    r->near = r->narrow && r->levels >= 2 && r->levels <= static_cast<uint32_t>(kNearLaneLevels) && r->scale_rows == 1 &&
              r->row_chunks < (1u << 24) && r->count[0] >= span && r->in[0] < (1u << 24) && r->out[0] < (1u << 24) &&
              r->scale_in[0] < (1u << 24) && r->scale_out[0] < (1u << 24);
}

// the same for the kernels that find each lane's row
// `unroll` > 0: the launch covers the whole tensor from tile 0 with tiles of kThreads * unroll chunks, so its
// workgroups may take the tiles in another order (LaneRows::order_*).
LaneRows lane_rows(const FlatArgs& a, int unroll = 0) {
    LaneRows r{};
    r.row_chunks = static_cast<uint32_t>(a.num_chunks);
    magic_of(r.row_chunks, &r.row_magic, &r.row_shift);
    r.total_chunks = static_cast<uint32_t>(a.rows * a.num_chunks);
    r.levels = a.lanes.levels;
    r.scale_rows = a.scale_rows > 1 ? a.scale_rows : 1u;
    magic_of(r.scale_rows, &r.scale_magic, &r.scale_shift);
    for (uint32_t l = 0; l < r.levels; l++) {
        r.count[l] = a.lanes.count[l];
        magic_of(r.count[l], &r.magic[l], &r.shift[l]);
        r.in[l] = a.lanes.in[l];
        r.out[l] = a.lanes.out[l];
        r.scale_in[l] = a.lanes.scale_in[l];
        r.scale_out[l] = a.lanes.scale_out[l];
    }
    set_narrow(&r);
    set_near(&r);
    const uint64_t tile_chunks = static_cast<uint64_t>(kThreads) * (unroll > 0 ? unroll : 1);
    const uint64_t run_chunks = static_cast<uint64_t>(r.count[0]) * r.row_chunks;  // chunks of one innermost run
    // measured on attention-shaped views (quantize / dequantize, us): reads of 512-byte rows gain (f32 rows of 128:
    // 143 -> 120, bf16 rows of 256: 86 -> 67), reads of 256-byte rows stay where they are, writes lose (68 -> 76)
    if (unroll > 0 && r.near && (r.row_chunks & (r.row_chunks - 1)) == 0 && r.row_chunks <= kThreads &&
        r.total_chunks % tile_chunks == 0 && r.count[0] % (tile_chunks / r.row_chunks) == 0) {
        uint32_t log2 = 0;
        while ((1u << log2) < r.row_chunks) log2++;
        r.whole_rows = 1 + log2;
    }
    const bool closer = r.levels >= 2 && r.in[1] < r.in[0] && r.row_chunks >= 32;
    if (unroll > 0 && r.near && closer && run_chunks % tile_chunks == 0 && r.count[1] > 1) {
        r.order_inner = static_cast<uint32_t>(run_chunks / tile_chunks);
        r.order_outer = r.count[1];
        magic_of(r.order_outer, &r.order_outer_magic, &r.order_outer_shift);
        magic_of(r.order_inner * r.order_outer, &r.order_slab_magic, &r.order_slab_shift);
    }
    return r;
}
inline uint32_t lanes_grid(const FlatArgs& a, int unroll) {
    const uint64_t per = static_cast<uint64_t>(kThreads) * unroll;
    return static_cast<uint32_t>((a.rows * a.num_chunks + per - 1) / per);
}

// One contiguous run of `chunks` chunks (< 2^31) as the lane-wise kernels see it: a single row.
LaneRows lane_rows_of_run(uint64_t chunks) {
    LaneRows r{};
    r.row_chunks = static_cast<uint32_t>(chunks);
    magic_of(r.row_chunks, &r.row_magic, &r.row_shift);
    r.total_chunks = r.row_chunks;
    r.levels = 1;
    r.scale_rows = 1;
    magic_of(1, &r.scale_magic, &r.scale_shift);
    r.count[0] = 1;
    magic_of(1, &r.magic[0], &r.shift[0]);
    r.narrow = 1;
    return r;
}
// Pitched rows (FlatArgs::rows > 1: groups of inner_rows rows) as the lane-wise kernels see them: one level for
// the rows of a group, one for the groups.  rows * num_chunks < 2^31.
LaneRows lane_rows_of_rows(const FlatArgs& a) {
    LaneRows r{};
    r.row_chunks = static_cast<uint32_t>(a.num_chunks);
    magic_of(r.row_chunks, &r.row_magic, &r.row_shift);
    r.total_chunks = static_cast<uint32_t>(a.rows * a.num_chunks);
    r.scale_rows = a.scale_rows > 1 ? a.scale_rows : 1u;
    magic_of(r.scale_rows, &r.scale_magic, &r.scale_shift);
    const uint64_t inner = a.inner_rows == 0 ? a.rows : a.inner_rows;
    r.levels = inner == a.rows ? 1 : 2;
    r.count[0] = static_cast<uint32_t>(inner);
    r.in[0] = a.in_pitch, r.out[0] = a.out_pitch, r.scale_in[0] = a.scale_in_pitch, r.scale_out[0] = a.scale_out_pitch;
    if (r.levels == 2) {
        r.count[1] = static_cast<uint32_t>(a.rows / inner);
        r.in[1] = a.in_outer, r.out[1] = a.out_outer, r.scale_in[1] = a.scale_in_outer, r.scale_out[1] = a.scale_out_outer;
    }
    for (uint32_t l = 0; l < r.levels; l++) magic_of(r.count[l], &r.magic[l], &r.shift[l]);
    set_narrow(&r);
    set_near(&r);
    return r;
}

constexpr uint64_t kKeepOutputBytes = 192ull << 20;  // QuantParams::keep: outputs up to this size
QuantParams quant_params(const Range& r) {
    QuantParams p;
    p.lo = r.lo;
    p.hi = r.hi;
    p.width = r.hi - r.lo;
    p.rwidth = 1.0f / p.width;  // IEEE division on the host: correctly rounded
    p.unrounded = r.unrounded;
    return p;
}

// How a flat launch is cut up.  The kernels over whole tiles check no bounds and exist for f32 parameters (a
// contiguous run, or pitched rows of whole steps) and for parameters typed like the float tensor, `f_dtype` (a
// contiguous run); everything else is the lane-wise kernel's:
//   `whole(grid, begin)`                       tiles [begin, begin + grid) of the run / of the rows' steps
//   `lanes(rows, tile_begin, grid, offsets)`   lane by lane; `offsets` = chunks / scales to advance the base
//                                              pointers by (a contiguous run only)
struct RunOffsets {
    uint64_t chunks;  // 16-byte chunks of the float tensor
};
template <class WholeFn, class LanesFn>
hipError_t launch_flat(const FlatArgs& a, int f_dtype, int unroll, WholeFn whole, LanesFn lanes) {
    const uint64_t tile = static_cast<uint64_t>(kThreads) * unroll;
    const bool p32 = a.param_dtype == CQ_F32;
    const int group = group_of(f_dtype, a.block);
    hipError_t e = hipSuccess;
    if (a.lanes.levels > 0) {
        lanes(lane_rows(a, unroll), 0u, lanes_grid(a, unroll), RunOffsets{0});
        return hipGetLastError();
    }
    if (a.rows > 1) {
        const LaneRows lr = lane_rows_of_rows(a);
        const uint32_t tiles = static_cast<uint32_t>((static_cast<uint64_t>(lr.total_chunks) + tile - 1) / tile);
        // whole steps: a tile is `unroll` steps in both numberings, so the ragged last tile can go lane by lane
        const uint32_t full = p32 && a.any_group == 0 && !a.lanes_only && whole_steps_for(group) && a.num_chunks % kThreads == 0
                                  ? static_cast<uint32_t>(lr.total_chunks / tile) : 0u;
        if (full > 0) {
            whole(full, 0ull);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
        if (full < tiles) {
            lanes(lr, full, tiles - full, RunOffsets{0});
            e = hipGetLastError();
        }
        return e;
    }
    // one contiguous run
    const uint64_t full = (p32 || a.param_dtype == f_dtype) && a.any_group == 0 && !a.lanes_only && whole_tiles_for(group) ? a.num_chunks / tile : 0;
    if (full > 0) {
        whole(static_cast<uint32_t>(full), 0ull);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    // the rest lane by lane, in pieces the 32-bit chunk numbers of those kernels can hold: a multiple of every tile and
    // every power-of-two block, or of whole blocks and whole words of codes
    const uint64_t piece = a.any_group == 0 ? (1ull << 30) : (1ull << 30) / (4ull * a.any_group) * (4ull * a.any_group);
    for (uint64_t begin = full * tile; begin < a.num_chunks; begin += piece) {
        const uint64_t n = a.num_chunks - begin < piece ? a.num_chunks - begin : piece;
        lanes(lane_rows_of_run(n), 0u, static_cast<uint32_t>((n + tile - 1) / tile), RunOffsets{begin});
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    return e;
}

template <class F, int kBits, int kGroup, int kSrc, bool kWide, int kEnc>
hipError_t quantize_launch_src(hipStream_t s, ScaleSource src, const FlatArgs& a) {
    // scale sources that exist: per-block launches compute the scale or read the
    // input-typed tensor; per-tensor launches read it or finish the grid reduction
    if constexpr ((kGroup == 0 && (kSrc == kScaleDynamic || kSrc == kScaleStored)) || (kGroup != 0 && kSrc == kScalePartials)) {
        return hipErrorInvalidValue;
    } else {
        // stored scales are read back by the second pass of a two-launch dynamic quantize, which runs lane by lane only
        if (kSrc == kScaleStored && a.lanes.levels == 0) return hipErrorInvalidValue;
        auto in = static_cast<const char*>(a.input);
        auto out = static_cast<char*>(a.output);
        QuantParams qp = quant_params(a.range);
        [[maybe_unused]] constexpr uint64_t kOutChunk = F::kPerChunk * kBits / 8;  // stored bytes per chunk
        // Codes that fit the 256 MB Infinity Cache with room to spare are stored to stay there for whoever reads
        // them next: on 147 MB of codes and scales (bf16 [28672, 8192], 4-bit, blocks of 32) a dequantize right
        // behind this launch takes 79 us instead of 96 us, the launch itself 0 - 3 % longer (up to 6 % on smaller
        // tensors).  Larger outputs stream past the caches.
        {
            const uint64_t chunks = a.num_chunks * (a.rows > 1 ? a.rows : 1);
            const uint64_t scales = kGroup == 0 ? 0 : chunks / (a.any_group != 0 ? a.any_group : kGroup) * (a.param_dtype == CQ_F32 ? 4 : 2);
            qp.keep = chunks * kOutChunk + scales <= kKeepOutputBytes ? 1u : 0u;
        }
        // bytes per scale of the two scale tensors (per-tensor launches and the partials never move their pointers)
        [[maybe_unused]] const uint64_t scale_in_bytes = kGroup == 0 ? 0 : (kSrc == kScaleStored ? (a.param_dtype == CQ_F32 ? 4 : 2) : F::kBytes);
        [[maybe_unused]] const uint64_t scale_out_bytes = kGroup == 0 ? 0 : (a.param_dtype == CQ_F32 ? 4 : 2);
        [[maybe_unused]] const uint64_t div = kGroup == 0 ? 1 : (a.any_group != 0 ? a.any_group : kGroup);  // chunks per scale
#if CQ_TU_SAME
        // this object: the whole tiles of a contiguous run, parameters typed like the tensor
        if constexpr (kSrc != kScaleStored && F::kBytes == 2 && !kWide && whole_tiles_for(kGroup)) {
            hipLaunchKernelGGL((quantize_flat_kernel<F, kBits, kGroup, kSrc, kWide, kUnrollQ, kThreads, kEnc, F::kDtype>),
                               dim3(a.whole_grid), dim3(kThreads), 0, s, reinterpret_cast<const u32x4*>(in),
                               reinterpret_cast<uint32_t*>(out), a.scale_in, a.scale_out, 0ull,
                               static_cast<uint64_t>(a.whole_grid) * kThreads * kUnrollQ, qp, a.num_partials);
            return hipGetLastError();
        } else {
            return hipErrorInvalidValue;
        }
#else
        hipError_t same = hipSuccess;
        const hipError_t e = launch_flat(
            a, F::kDtype, kUnrollQ,
            [&](uint32_t grid, uint64_t) {
                if constexpr (kSrc != kScaleStored && !kWide) {  // (fields that wrap: lane by lane only)
                    if (a.param_dtype != CQ_F32) {  // a contiguous run, parameters typed like the tensor
                        FlatArgs b = a;
                        b.whole_grid = grid;
                        same = quantize_flat_same<F>(kSrc == kScaleGivenF, s, kBits, src, b);
                    } else if (a.rows > 1) {
                        if constexpr (whole_steps_for(kGroup))
                            hipLaunchKernelGGL((quantize_flat_rows_kernel<F, kBits, kGroup, kSrc, kWide, kUnrollQ, kThreads, kEnc>),
                                               dim3(grid), dim3(kThreads), 0, s, reinterpret_cast<const u32x4*>(in),
                                               reinterpret_cast<uint32_t*>(out), a.scale_in, a.scale_out, 0u, qp, a.num_partials,
                                               flat_rows(a));
                    } else {
                        if constexpr (whole_tiles_for(kGroup))
                            hipLaunchKernelGGL((quantize_flat_kernel<F, kBits, kGroup, kSrc, kWide, kUnrollQ, kThreads, kEnc>),
                                               dim3(grid), dim3(kThreads), 0, s, reinterpret_cast<const u32x4*>(in),
                                               reinterpret_cast<uint32_t*>(out), a.scale_in, a.scale_out, 0ull,
                                               static_cast<uint64_t>(grid) * kThreads * kUnrollQ, qp, a.num_partials);
                    }
                }
            },
            [&](const LaneRows& rows, uint32_t tile_begin, uint32_t grid, RunOffsets off) {
                const uint64_t scales = off.chunks / div;
                const void* scale_in = a.scale_in == nullptr ? nullptr : static_cast<const char*>(a.scale_in) + scales * scale_in_bytes;
                void* scale_out = a.scale_out == nullptr ? nullptr : static_cast<char*>(a.scale_out) + scales * scale_out_bytes;
                hipLaunchKernelGGL((quantize_flat_lanes_kernel<F, kBits, lanes_group(kGroup), kSrc, kWide, kUnrollQ, kThreads, kEnc>),
                                   dim3(grid), dim3(kThreads), 0, s, reinterpret_cast<const u32x4*>(in + off.chunks * 16),
                                   reinterpret_cast<uint32_t*>(out + off.chunks * kOutChunk), scale_in, scale_out,
                                   a.param_dtype, qp, a.num_partials, tile_begin, with_group(rows, kGroup, a.any_group));
            });
        return e != hipSuccess ? e : same;
#endif
    }
}

// kGiven: the translation unit holds the kernels that read given scales, or those that produce
// the scale themselves (the two sets are compiled apart: together they take minutes).
template <class F, int kBits, int kGroup, bool kWide, int kEnc, bool kGiven>
hipError_t quantize_launch_enc(hipStream_t s, ScaleSource src, const FlatArgs& a) {
    if constexpr (kGiven) {
        if (src == ScaleSource::Given && a.scale_in_dtype == F::kDtype)  // given scales are typed like the input
            return quantize_launch_src<F, kBits, kGroup, kScaleGivenF, kWide, kEnc>(s, src, a);
        if (src == ScaleSource::Stored) return quantize_launch_src<F, kBits, kGroup, kScaleStored, kWide, kEnc>(s, src, a);
    } else {
        if (src == ScaleSource::Dynamic) return quantize_launch_src<F, kBits, kGroup, kScaleDynamic, kWide, kEnc>(s, src, a);
        if (src == ScaleSource::Partials) return quantize_launch_src<F, kBits, kGroup, kScalePartials, kWide, kEnc>(s, src, a);
    }
    return hipErrorInvalidValue;
}

template <class F, int kBits, int kGroup, bool kGiven>
hipError_t quantize_launch(hipStream_t s, ScaleSource src, const FlatArgs& a) {
    switch (a.encoding) {
        case kEncInt:
            // value ranges wider than their field (E4M3 / E5M2 in the U32 store): fields wrap like the reference's
            // `i32 & mask` (src/quantize.rs:75), lane by lane only (FlatArgs::lanes_only, set by the caller)
            if (fields_wrap(a)) {
                if constexpr (kBits == 8) {
                    if (!a.lanes_only) return hipErrorInvalidValue;
                    return quantize_launch_enc<F, 8, kGroup, true, kEncInt, kGiven>(s, src, a);
                } else {
                    return hipErrorInvalidValue;
                }
            }
            return quantize_launch_enc<F, kBits, kGroup, false, kEncInt, kGiven>(s, src, a);
        case kEncE4M3:
            if constexpr (kBits == 8) return quantize_launch_enc<F, 8, kGroup, false, kEncE4M3, kGiven>(s, src, a);
            break;
        case kEncE5M2:
            if constexpr (kBits == 8) return quantize_launch_enc<F, 8, kGroup, false, kEncE5M2, kGiven>(s, src, a);
            break;
        case kEncE2M1:
            if constexpr (kBits == 4) return quantize_launch_enc<F, 4, kGroup, false, kEncE2M1, kGiven>(s, src, a);
            break;
    }
    return hipErrorInvalidValue;
}

#define CQ_SWITCH_GROUP(G, ...)                          \
    switch (G) {                                         \
        case 0: { constexpr int kG = 0; __VA_ARGS__; }   \
        case 1: { constexpr int kG = 1; __VA_ARGS__; }   \
        case 2: { constexpr int kG = 2; __VA_ARGS__; }   \
        case 4: { constexpr int kG = 4; __VA_ARGS__; }   \
        case 8: { constexpr int kG = 8; __VA_ARGS__; }   \
        case 16: { constexpr int kG = 16; __VA_ARGS__; } \
        case 32: { constexpr int kG = 32; __VA_ARGS__; } \
        default: return hipErrorInvalidValue;            \
    }

#define CQ_SWITCH_BITS(B, ...)                          \
    switch (B) {                                        \
        case 2: { constexpr int kB = 2; __VA_ARGS__; }  \
        case 4: { constexpr int kB = 4; __VA_ARGS__; }  \
        case 8: { constexpr int kB = 8; __VA_ARGS__; }  \
        default: return hipErrorInvalidValue;           \
    }

#define CQ_SWITCH_DTYPE(D, ...)                              \
    switch (D) {                                             \
        case CQ_F32: { using kF = F32; __VA_ARGS__; }        \
        case CQ_BF16: { using kF = BF16; __VA_ARGS__; }      \
        case CQ_F16: { using kF = F16; __VA_ARGS__; }        \
        default: return hipErrorInvalidValue;                \
    }

}  // namespace
}  // namespace cq
