// Row kernels: quantize / dequantize / block abs-max for every layout whose last
// dimension is contiguous but which the flat streaming kernels cannot take:
// N-D blocks (e.g. 128 x 128), block sizes that are not a power-of-two number of
// lanes (e.g. 24), strided scale tensors, pitched or sliced rows, permuted leading
// dimensions.  Same arithmetic as the flat kernels (cq_device.hpp), same addressing
// rules as the reference's layouts (crates/cubek-quant/src/layout/scales.rs:144-194).
//
// A workgroup covers TR rows x TJ units (TR * TJ = 256, TJ a power of two chosen on
// the host from the row length).  A unit is the smallest run of elements that is
// whole on both sides: max(values per stored word, values per 16-byte chunk).  Each
// thread decomposes its row index once (strides and block coordinates of the
// leading dimensions) and then walks kUnits units of that row; loads and stores are
// 16 bytes of floats and whole 32-bit words.
//
//   quantize_rows_kernel / dequantize_rows_kernel   scales given / stored
//   scales_rows_kernel        abs-max of BR x BC blocks -> scales
//   quantize_blocks_kernel    abs-max + scale + quantize of BR x BC blocks in one launch
//   absmax_rows_kernel        per-tensor abs-max partials over strided rows
#include "cq_device.hpp"
#include "cq_internal.hpp"

namespace cq {
namespace {

constexpr int kThreads = 256;

template <class F, int kBits>
struct Unit {
    static constexpr int kN = F::kPerChunk;           // values per 16-byte chunk
    static constexpr int kNq = 32 / kBits;            // values per stored word
    static constexpr int kV = kNq > kN ? kNq : kN;    // values per unit
    static constexpr int kChunks = kV / kN;
    static constexpr int kWords = kV / kNq;
    static constexpr int kUnits = kChunks >= 4 ? 2 : 4;  // units per thread
};

// What a thread knows about its row.
struct RowPos {
    uint64_t f, v, sa, sb;  // offsets: floats (elements), stored (words), scale_in, scale_out
    bool start;             // every leading coordinate sits on a block start
    bool live;
};

__device__ __forceinline__ RowPos row_pos(const RowArgs& a, uint32_t row) {
    RowPos r{0, 0, 0, 0, true, row < a.rows};
    uint32_t rem = r.live ? row : 0;
    for (int d = static_cast<int>(a.rank) - 2; d >= 0; d--) {
        // the outermost coordinate is what is left; integer division is a long instruction sequence
        const uint32_t c = d == 0 ? rem : rem % a.shape[d];
        if (d != 0) rem /= a.shape[d];
        r.f += static_cast<uint64_t>(c) * a.fstride[d];
        r.v += static_cast<uint64_t>(c) * a.vstride[d];
        if (a.tensor_level) {
            r.start = r.start && c == 0;
        } else if (a.block[d] == 1) {
            r.sa += static_cast<uint64_t>(c) * a.sa[d];
            r.sb += static_cast<uint64_t>(c) * a.sb[d];
        } else {
            const uint32_t cb = c / a.block[d];
            r.sa += static_cast<uint64_t>(cb) * a.sa[d];
            r.sb += static_cast<uint64_t>(cb) * a.sb[d];
            r.start = r.start && c == cb * a.block[d];
        }
    }
    return r;
}

// Scale offsets and block-start flag of the unit that begins at column `e`.
struct ScaleAt {
    uint64_t a, b;
    bool start;
};
__device__ __forceinline__ ScaleAt scale_at(const RowArgs& a, const RowPos& r, uint32_t e) {
    if (a.tensor_level) return ScaleAt{0, 0, r.start && e == 0};
    const int last = static_cast<int>(a.rank) - 1;
    const uint32_t bc = a.block[last];
    const uint32_t cb = a.bc_shift >= 0 ? e >> a.bc_shift : e / bc;
    return ScaleAt{r.sa + static_cast<uint64_t>(cb) * a.sa[last], r.sb + static_cast<uint64_t>(cb) * a.sb[last],
                   r.start && e == cb * bc};
}

template <class F, int kBits, bool kWide, int kEnc>
__global__ __launch_bounds__(kThreads) void quantize_rows_kernel(RowArgs a) {
    using U = Unit<F, kBits>;
    constexpr int kN = U::kN;
    const uint32_t tj = 1u << a.tj_log2;
    const uint32_t row = blockIdx.x * (kThreads >> a.tj_log2) + (threadIdx.x >> a.tj_log2);
    const uint32_t jl = threadIdx.x & (tj - 1);
    const RowPos r = row_pos(a, row);
    const u32x4* in = static_cast<const u32x4*>(a.input);
    uint32_t* out = static_cast<uint32_t*>(a.output);

    u32x4 raw[U::kUnits][U::kChunks];
    float s_f[U::kUnits];
    ScaleAt sp[U::kUnits];
#pragma unroll
    for (int u = 0; u < U::kUnits; u++) {
        uint32_t j = (blockIdx.y * U::kUnits + u) * tj + jl;
        j = j < a.units_per_row ? j : a.units_per_row - 1;  // clamp instead of branching around loads
        const uint32_t e = j * U::kV;
        sp[u] = scale_at(a, r, e);
        s_f[u] = load_dtype(a.scale_in_dtype, a.scale_in, sp[u].a);
#pragma unroll
        for (int i = 0; i < U::kChunks; i++) raw[u][i] = stream_load(in + (r.f + e) / kN + i);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U::kUnits; u++) {
        const uint32_t j = (blockIdx.y * U::kUnits + u) * tj + jl;
        const bool live = r.live && j < a.units_per_row;
        // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first element
        const float s_fs = round_to_dtype(a.param_dtype, s_f[u]);
        if (a.scale_out != nullptr && live && sp[u].start) store_dtype(a.param_dtype, a.scale_out, sp[u].b, s_fs);
        const float d = F::round(s_fs);
        const bool tame = divisor_is_tame(d);
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < U::kChunks; i++) {
            float v[kN], qn[kN];
            F::unpack(raw[u][i], v);
            quantize_codes<F, kN, kEnc>(v, d, tame, a.range.lo, a.range.hi, a.range.unrounded != 0, qn);
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
        if (live) {
            uint32_t* dst = out + r.v + static_cast<uint64_t>(j) * U::kWords;
            stream_store(w[0], dst);
            if constexpr (U::kWords == 2) stream_store(w[1], dst + 1);
        }
    }
}

template <class F, int kBits, int kEnc>
__global__ __launch_bounds__(kThreads) void dequantize_rows_kernel(RowArgs a) {
    using U = Unit<F, kBits>;
    constexpr int kN = U::kN;
    const uint32_t tj = 1u << a.tj_log2;
    const uint32_t row = blockIdx.x * (kThreads >> a.tj_log2) + (threadIdx.x >> a.tj_log2);
    const uint32_t jl = threadIdx.x & (tj - 1);
    const RowPos r = row_pos(a, row);
    const uint32_t* in = static_cast<const uint32_t*>(a.input);
    u32x4* out = static_cast<u32x4*>(a.output);

    uint32_t w[U::kUnits][U::kWords];
    float sc[U::kUnits];
#pragma unroll
    for (int u = 0; u < U::kUnits; u++) {
        uint32_t j = (blockIdx.y * U::kUnits + u) * tj + jl;
        j = j < a.units_per_row ? j : a.units_per_row - 1;
        const ScaleAt sp = scale_at(a, r, j * U::kV);
        sc[u] = F::round(load_dtype(a.param_dtype, a.scale_in, sp.a));  // Line::cast_from(scale)
#pragma unroll
        for (int k = 0; k < U::kWords; k++) w[u][k] = stream_load(in + r.v + static_cast<uint64_t>(j) * U::kWords + k);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U::kUnits; u++) {
        const uint32_t j = (blockIdx.y * U::kUnits + u) * tj + jl;
        float y[U::kV];
#pragma unroll
        for (int k = 0; k < U::kWords; k++) decode_fields<kEnc, kBits, U::kNq>(w[u][k], y + k * U::kNq);
#pragma unroll
        for (int i = 0; i < U::kV; i++) y[i] = sc[u] * y[i];
        if (r.live && j < a.units_per_row) {
#pragma unroll
            for (int i = 0; i < U::kChunks; i++)
                stream_store(F::pack(y + i * kN), out + (r.f + static_cast<uint64_t>(j) * U::kV) / kN + i);  // pack rounds to F
        }
    }
}

// Abs-max of every block [BR rows x BC columns] (blocks extend over the last two
// dimensions only) -> scale typed `out_dtype` through the strides `sb`.
// Thread = (block row, 16-byte chunk column); it walks the BR rows of its block
// row, then the chunk columns of one block meet in LDS.
template <class F>
__global__ __launch_bounds__(kThreads) void scales_rows_kernel(RowArgs a, int out_dtype, uint32_t block_rows,
                                                               uint32_t chunks_per_block, uint32_t tj_eff) {
    constexpr int kN = F::kPerChunk;
    constexpr int kUnroll = 4;
    __shared__ float lds[kThreads];
    const int last = static_cast<int>(a.rank) - 1;
    const uint32_t tj = 1u << a.tj_log2;
    const uint32_t rbi = blockIdx.x * (kThreads >> a.tj_log2) + (threadIdx.x >> a.tj_log2);
    const uint32_t jl = threadIdx.x & (tj - 1);
    const uint32_t jc = blockIdx.y * tj_eff + jl;
    const uint32_t chunks_per_row = a.shape[last] / kN;
    const uint32_t br = a.rank >= 2 ? a.block[last - 1] : 1u;
    const bool live = rbi < block_rows && jl < tj_eff && jc < chunks_per_row;
    // the block row's first row, as a flattened row index
    const RowPos r = row_pos(a, live ? rbi * br : 0);
    float amax = 0.0f;
    if (live) {
        const u32x4* p = static_cast<const u32x4*>(a.input) + r.f / kN + jc;
        const uint64_t pitch = a.rank >= 2 ? a.fstride[last - 1] / kN : 0;
        for (uint32_t r0 = 0; r0 < br; r0 += kUnroll) {
            u32x4 raw[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                raw[u] = u32x4{0, 0, 0, 0};
                if (r0 + u < br) raw[u] = stream_load(p + (r0 + u) * pitch);  // the same for the whole workgroup
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                float v[kN];
                F::unpack(raw[u], v);
#pragma unroll
                for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
            }
        }
    }
    lds[threadIdx.x] = amax;
    __syncthreads();
    if (live && jc % chunks_per_block == 0) {
        for (uint32_t k = 1; k < chunks_per_block; k++) amax = fmaxf(amax, lds[threadIdx.x + k]);
        const float s = F::round(scale_from_absmax(amax, a.range.hi - a.range.lo));
        store_dtype(out_dtype, a.scale_out, r.sb + static_cast<uint64_t>(jc / chunks_per_block) * a.sb[last],
                    round_to_dtype(out_dtype, s));
    }
}

// Fused dynamic quantize for blocks of BR rows x BC columns (BC a whole number of
// chunks): abs-max, scale, out_scale and codes in one launch that reads the input
// once.  A tile is what one workgroup holds at a time: TJ chunk columns (x kCols tiles
// side by side) x (256 / TJ) row phases; PH phases share a block row and each keeps
// every PH-th row of it in registers (at most kRows 16-byte chunks), so small BR puts
// several block rows into one tile.  The abs-max meets across the chunk columns of a
// block by DPP (power-of-two widths; other widths use only the lanes that hold whole
// blocks and meet in LDS) and across the phases in LDS.
// One workgroup per tile.  (A persistent variant that loaded tile i+1 before working on tile i
// was slower at every block shape: 44 us against 39-41 us on 128 x 128 blocks of a bf16
// [8192, 8192], 144 us against 129 us on [28672, 8192].)
template <int kLog2>
__device__ __forceinline__ float group_max_log2(float v, uint32_t log2) {
    if constexpr (kLog2 > 5) {
        return v;
    } else {
        if (log2 == kLog2) return group_max<(1 << kLog2)>(v);
        return group_max_log2<kLog2 + 1>(v, log2);
    }
}

struct BlocksGeom {
    uint32_t cpb, cpb_log2;  // chunks per block along the row; its log2, or 32 when not a power of two
    uint32_t tj_log2, tj_eff;  // lanes along the row, and how many of them hold whole blocks
    uint32_t ph_per_block, per_group, rows_per_thread;
    uint32_t num_block_rows, col_groups, tiles;
};

template <class F, int kBits, bool kWide, int kEnc, int kRows, int kCols>
__global__ __launch_bounds__(kThreads) void quantize_blocks_kernel(RowArgs a, BlocksGeom g, QuantParams qp) {
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    __shared__ float lds[kCols][kThreads];
    const int last = static_cast<int>(a.rank) - 1;
    const uint32_t tj = 1u << g.tj_log2;
    const uint32_t ph = threadIdx.x >> g.tj_log2, jl = threadIdx.x & (tj - 1);
    const uint32_t bsub = ph / g.ph_per_block, pin = ph % g.ph_per_block;
    const uint32_t chunks_per_row = a.shape[last] / kN;
    const uint32_t br = a.rank >= 2 ? a.block[last - 1] : 1u;
    const uint64_t pitch_f = a.rank >= 2 ? a.fstride[last - 1] / kN : 0;
    const uint64_t pitch_v = a.rank >= 2 ? a.vstride[last - 1] : 0;

    // this thread's place in tile t: offsets of its block row, its first chunk column
    struct Pos {
        uint64_t f, v, sb;
        uint32_t jc0;
        bool rows_live;
    };
    auto locate = [&](uint32_t t) {
        const uint32_t rg = t / g.col_groups, cg = t - rg * g.col_groups;
        const uint32_t rbi = rg * g.per_group + bsub;
        Pos p;
        p.rows_live = bsub < g.per_group && rbi < g.num_block_rows;
        const RowPos r = row_pos(a, p.rows_live ? rbi * br : 0);
        p.f = r.f / kN;
        p.v = r.v;
        p.sb = r.sb;
        p.jc0 = cg * (kCols * g.tj_eff) + jl;
        return p;
    };
    auto load = [&](const Pos& p, u32x4 (&raw)[kCols][kRows]) {
        // this thread's rows lie ph_per_block rows apart: one 64-bit product, then steps of a tile-wide constant
        const u32x4* src = static_cast<const u32x4*>(a.input) + p.f + pin * pitch_f;
        const uint64_t row_step = g.ph_per_block * pitch_f;
#pragma unroll
        for (int c = 0; c < kCols; c++) {
            const uint32_t jc = p.jc0 + c * g.tj_eff;
            const u32x4* at = src + jc;
#pragma unroll
            for (int k = 0; k < kRows; k++) {
                const uint32_t rr = pin + k * g.ph_per_block;
                raw[c][k] = u32x4{0, 0, 0, 0};
                if (p.rows_live && jl < g.tj_eff && jc < chunks_per_row && rr < br) raw[c][k] = stream_load(at);
                at += row_step;
            }
        }
    };

    const Pos pos = locate(blockIdx.x);
    u32x4 raw[kCols][kRows];
    load(pos, raw);
    {
        float amax[kCols];
#pragma unroll
        for (int c = 0; c < kCols; c++) {
            amax[c] = 0.0f;
#pragma unroll
            for (int k = 0; k < kRows; k++) {
                float v[kN];
                F::unpack(raw[c][k], v);
#pragma unroll
                for (int i = 0; i < kN; i++) amax[c] = fmaxf(amax[c], fabsf(v[i]));  // NaN elements drop out
            }
            amax[c] = group_max_log2<0>(amax[c], g.cpb_log2);  // over the chunk columns of a power-of-two block
            lds[c][threadIdx.x] = amax[c];
        }
        __syncthreads();

#pragma unroll
        for (int c = 0; c < kCols; c++) {
            const uint32_t jc = pos.jc0 + c * g.tj_eff;
            const bool live = pos.rows_live && jl < g.tj_eff && jc < chunks_per_row;  // the same for every lane of a word
            const bool pow2 = g.cpb_log2 < 32;
            // first lane and number of LDS entries of this block in a phase: after the DPP step every
            // lane of a power-of-two block holds its maximum; other widths meet here, entry by entry
            const uint32_t lane0 = pow2 ? jl : (jl < g.tj_eff ? jl / g.cpb * g.cpb : 0);
            const uint32_t entries = pow2 ? 1u : g.cpb;
            if (bsub < g.per_group)  // phases beyond the last whole block row hold nothing
                for (uint32_t p = 0; p < g.ph_per_block; p++)
                    for (uint32_t k = 0; k < entries; k++)
                        amax[c] = fmaxf(amax[c], lds[c][((bsub * g.ph_per_block + p) << g.tj_log2) + lane0 + k]);
            const float s32 =
                absmax_is_tame(amax[c]) ? scale_from_absmax_tame(amax[c], qp) : scale_from_absmax(amax[c], qp.width);
            const float s_fs = round_to_dtype(a.param_dtype, F::round(s32));
            const uint32_t block_col = pow2 ? jc >> g.cpb_log2 : jc / g.cpb;
            if (live && pin == 0 && jc == block_col * g.cpb)
                store_dtype(a.param_dtype, a.scale_out, pos.sb + static_cast<uint64_t>(block_col) * a.sb[last], s_fs);
            const float d = F::round(s_fs);
            const bool tame = divisor_is_tame(d);
            if (!live) continue;
            uint32_t* dst = static_cast<uint32_t*>(a.output) + pos.v + pin * pitch_v;
            const uint64_t out_step = g.ph_per_block * pitch_v;
#pragma unroll
            for (int k = 0; k < kRows; k++, dst += out_step) {
                const uint32_t rr = pin + k * g.ph_per_block;
                const bool row_live = rr < br;  // the same for every lane of a word
                float v[kN], qn[kN];
                F::unpack(raw[c][k], v);
                quantize_codes<F, kN, kEnc>(v, d, tame, qp.lo, qp.hi, qp.unrounded != 0, qn);
                uint32_t w[2] = {0, 0};
                if constexpr (kEnc == kEncInt)
                    pack_chunk_neg<kBits, kN, kWide>(qn, w);
                else
                    encode_chunk<kEnc, kN>(qn, w);
                if constexpr (kChunkBits == 64) {
                    if (row_live) {
                        stream_store(w[0], dst + 2 * static_cast<uint64_t>(jc));
                        stream_store(w[1], dst + 2 * static_cast<uint64_t>(jc) + 1);
                    }
                } else if constexpr (kChunkBits == 32) {
                    if (row_live) stream_store(w[0], dst + jc);
                } else {
                    // neighbouring lanes (same row) hold the other parts of the word
                    constexpr int kLanesPerWord = 32 / kChunkBits;
                    const uint32_t sub = jc & (kLanesPerWord - 1);
                    const uint32_t word = group_or<kLanesPerWord>(w[0] << (sub * kChunkBits));
                    if (row_live && sub == 0) stream_store(word, dst + jc / kLanesPerWord);
                }
            }
        }
    }
}

// Per-tensor abs-max, pass 1, over strided rows: gridDim.x <= kMaxPartials workgroups of 1024
// threads stride over the (row tile, chunk tile) pairs; one f32 partial per workgroup.  A
// maximum does not mind seeing an element twice: indices beyond the end are clamped to the
// last tile / row / chunk instead of guarding every load.
constexpr int kAbsmaxThreads = 1024;
template <class F>
__global__ __launch_bounds__(kAbsmaxThreads) void absmax_rows_kernel(RowArgs a, float* __restrict__ partials,
                                                                     uint32_t row_tiles, uint32_t col_tiles) {
    constexpr int kN = F::kPerChunk;
    __shared__ float lds[kAbsmaxThreads / kWave];
    const int last = static_cast<int>(a.rank) - 1;
    const uint32_t tj = 1u << a.tj_log2;
    const uint32_t chunks_per_row = a.shape[last] / kN;
    const uint32_t last_row = static_cast<uint32_t>(a.rows - 1);
    const u32x4* in = static_cast<const u32x4*>(a.input);
    constexpr int kUnroll = 4;  // tiles in flight per thread
    const uint32_t tiles = row_tiles * col_tiles;  // the launcher keeps it below 2^32
    float amax = 0.0f;
    for (uint32_t t0 = blockIdx.x; t0 < tiles; t0 += gridDim.x * kUnroll) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            uint32_t t = t0 + u * gridDim.x;
            t = t < tiles ? t : tiles - 1;
            const uint32_t rt = t / col_tiles, ct = t - rt * col_tiles;
            uint32_t row = rt * (kAbsmaxThreads >> a.tj_log2) + (threadIdx.x >> a.tj_log2);
            uint32_t jc = ct * tj + (threadIdx.x & (tj - 1));
            row = row < last_row ? row : last_row;
            jc = jc < chunks_per_row ? jc : chunks_per_row - 1;
            const RowPos r = row_pos(a, row);
            raw[u] = stream_load(in + r.f / kN + jc);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            float v[kN];
            F::unpack(raw[u], v);
#pragma unroll
            for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
        }
    }
    amax = group_max<kWave>(amax);
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kAbsmaxThreads / kWave; w++) amax = fmaxf(amax, lds[w]);
        partials[blockIdx.x] = amax;
    }
}

// lanes along the row: the smallest power of two that covers `units`, at most 256
uint32_t lanes_log2(uint64_t units) {
    uint32_t l = 0;
    while (l < 8 && (1ull << l) < units) l++;
    return l;
}

#define CQ_SWITCH_DTYPE(D, ...)                              \
    switch (D) {                                             \
        case CQ_F32: { using kF = F32; __VA_ARGS__; }        \
        case CQ_BF16: { using kF = BF16; __VA_ARGS__; }      \
        case CQ_F16: { using kF = F16; __VA_ARGS__; }        \
        default: return hipErrorInvalidValue;                \
    }

template <class F, int kBits>
dim3 unit_grid(RowArgs* a) {
    using U = Unit<F, kBits>;
    a->units_per_row = a->shape[a->rank - 1] / U::kV;
    a->tj_log2 = lanes_log2((a->units_per_row + U::kUnits - 1) / U::kUnits);
    // fewer lanes along the row (not below 64) where that leaves clearly fewer of them idle past the row end
    const auto covered = [&](uint32_t log2) {
        const uint64_t per = static_cast<uint64_t>(U::kUnits) << log2;
        return (a->units_per_row + per - 1) / per * per;
    };
    for (uint32_t l = a->tj_log2; l > 6; l--)
        if (covered(l - 1) * 10 <= covered(a->tj_log2) * 9) a->tj_log2 = l - 1;
    const uint32_t tr = kThreads >> a->tj_log2;
    const uint32_t per_group = U::kUnits << a->tj_log2;
    return dim3(static_cast<uint32_t>((a->rows + tr - 1) / tr), (a->units_per_row + per_group - 1) / per_group);
}

template <class F>
hipError_t quantize_rows(hipStream_t s, int bits, RowArgs a) {
    const bool wide = a.range.hi > 127.0f || a.range.lo < -128.0f;
#define CQ_LAUNCH(B, W, E)                                                                                    \
    {                                                                                                         \
        const dim3 grid = unit_grid<F, B>(&a);                                                                \
        hipLaunchKernelGGL((quantize_rows_kernel<F, B, W, E>), grid, dim3(kThreads), 0, s, a);                \
        return hipGetLastError();                                                                             \
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
hipError_t dequantize_rows(hipStream_t s, int bits, RowArgs a) {
#define CQ_LAUNCH(B, E)                                                                                       \
    {                                                                                                         \
        const dim3 grid = unit_grid<F, B>(&a);                                                                \
        hipLaunchKernelGGL((dequantize_rows_kernel<F, B, E>), grid, dim3(kThreads), 0, s, a);                 \
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

constexpr uint32_t kMaxRowsPerThread = 16;
constexpr uint32_t kPreferredRowsPerThread = 8;

// kRows x kCols chunks per thread: tall blocks keep their rows, flat ones take several
// column tiles so that a thread still has 4-16 loads in flight.
inline uint32_t blocks_cols_per_thread(uint32_t rows_per_thread) {
    return rows_per_thread <= 2 ? 4u : (rows_per_thread <= 4 ? 2u : 1u);
}

// Geometry of quantize_blocks_kernel for one launch; false when a block row does not fit
// the registers of one workgroup or there are too many tiles for 32-bit indices.
bool blocks_geom(uint32_t per_chunk, uint32_t bits, const RowArgs& a, BlocksGeom* g) {
    const uint32_t last = a.rank - 1;
    const uint32_t br = a.rank >= 2 ? a.block[last - 1] : 1u;
    const uint32_t chunks_per_row = a.shape[last] / per_chunk, cpb = a.block[last] / per_chunk;
    g->cpb = cpb;
    uint32_t cover_log2 = 0;  // lanes that cover one block
    while ((1u << cover_log2) < cpb) cover_log2++;
    g->cpb_log2 = (1u << cover_log2) == cpb ? cover_log2 : 32u;
    const uint32_t min_log2 = cover_log2 > 2 ? cover_log2 : 2;  // at least one block and one word
    // as many lanes along the row as the rows allow, while a block row still fits the registers
    uint32_t tj_log2 = lanes_log2(chunks_per_row);
    if (tj_log2 < min_log2) tj_log2 = min_log2;
    while (tj_log2 > min_log2 && br > kPreferredRowsPerThread * (kThreads >> tj_log2)) tj_log2--;
    // A thread takes 1-4 column tiles: narrower lanes (more rows per workgroup) while half the lanes
    // would still cover the row, and while that leaves clearly fewer idle lanes in the last column
    // group (rows of 128 chunks ran at a quarter of the lanes, rows of 1152 chunks at 56 %).
    const auto cols_at = [&](uint32_t log2) {
        const uint32_t phases = kThreads >> log2, ppb = br >= phases ? phases : br;
        return blocks_cols_per_thread((br + ppb - 1) / ppb) << log2;  // chunks one column group covers (all lanes in use)
    };
    const auto covered_at = [&](uint32_t log2) {
        const uint64_t per = cols_at(log2);
        return (chunks_per_row + per - 1) / per * per;
    };
    while (tj_log2 > min_log2 && cols_at(tj_log2 - 1) >= chunks_per_row) tj_log2--;
    for (uint32_t l = tj_log2; l > min_log2 && l > 6; l--)  // not below 64 lanes: runs of 1 KiB
        if (covered_at(l - 1) * 10 <= covered_at(tj_log2) * 9) tj_log2 = l - 1;
    const uint32_t phases = kThreads >> tj_log2;
    g->tj_log2 = tj_log2;
    // whole blocks and whole stored words only (lanes that share a word exchange their parts by lane number)
    const uint32_t chunk_bits = per_chunk * bits;
    const uint32_t word_lanes = chunk_bits >= 32 ? 1u : 32u / chunk_bits;
    uint32_t step = cpb;
    while (step % word_lanes) step += cpb;
    g->tj_eff = ((1u << tj_log2) / step) * step;
    if (g->tj_eff == 0) return false;
    g->ph_per_block = br >= phases ? phases : br;
    g->per_group = br >= phases ? 1u : phases / br;
    g->rows_per_thread = (br + g->ph_per_block - 1) / g->ph_per_block;
    if (g->rows_per_thread > kMaxRowsPerThread) return false;
    const uint64_t num_block_rows = a.rows / br;
    const uint32_t per_group_cols = blocks_cols_per_thread(g->rows_per_thread) * g->tj_eff;
    const uint64_t row_groups = (num_block_rows + g->per_group - 1) / g->per_group;
    g->num_block_rows = static_cast<uint32_t>(num_block_rows);
    g->col_groups = (chunks_per_row + per_group_cols - 1) / per_group_cols;
    const uint64_t tiles = row_groups * g->col_groups;
    g->tiles = static_cast<uint32_t>(tiles);
    return tiles < (1ull << 31);
}

template <class F, int kBits, bool kWide, int kEnc, int kRows, int kCols>
hipError_t quantize_blocks_variant(hipStream_t s, const RowArgs& a, const BlocksGeom& g, const QuantParams& qp) {
    hipLaunchKernelGGL((quantize_blocks_kernel<F, kBits, kWide, kEnc, kRows, kCols>), dim3(g.tiles), dim3(kThreads), 0, s, a,
                       g, qp);
    return hipGetLastError();
}

template <class F, int kBits, bool kWide, int kEnc>
hipError_t quantize_blocks_rows(hipStream_t s, const RowArgs& a, const BlocksGeom& g, const QuantParams& qp) {
    if (g.rows_per_thread <= 1) return quantize_blocks_variant<F, kBits, kWide, kEnc, 1, 4>(s, a, g, qp);
    if (g.rows_per_thread <= 2) return quantize_blocks_variant<F, kBits, kWide, kEnc, 2, 4>(s, a, g, qp);
    if (g.rows_per_thread <= 4) return quantize_blocks_variant<F, kBits, kWide, kEnc, 4, 2>(s, a, g, qp);
    // f32: the eight-row variant compiles to 120 registers (half the waves per SIMD: 29 % of HBM peak), the
    // sixteen-row one to 52, and rows beyond a block's are neither loaded nor stored
    if (g.rows_per_thread <= 8 && F::kBytes != 4) return quantize_blocks_variant<F, kBits, kWide, kEnc, 8, 1>(s, a, g, qp);
    return quantize_blocks_variant<F, kBits, kWide, kEnc, 16, 1>(s, a, g, qp);
}

template <class F>
hipError_t quantize_blocks(hipStream_t s, int bits, const RowArgs& a) {
    BlocksGeom g;
    if (!blocks_geom(F::kPerChunk, static_cast<uint32_t>(bits), a, &g)) return hipErrorInvalidValue;
    if (g.tiles == 0) return hipSuccess;
    QuantParams qp;
    qp.lo = a.range.lo;
    qp.hi = a.range.hi;
    qp.width = a.range.hi - a.range.lo;
    qp.rwidth = 1.0f / qp.width;  // IEEE division on the host: correctly rounded
    qp.unrounded = a.range.unrounded;
    const bool wide = a.range.hi > 127.0f || a.range.lo < -128.0f;
    switch (a.encoding) {
        case kEncInt:
            if (bits == 2) return quantize_blocks_rows<F, 2, false, kEncInt>(s, a, g, qp);
            if (bits == 4) return quantize_blocks_rows<F, 4, false, kEncInt>(s, a, g, qp);
            if (bits == 8 && wide) break;  // ranges wider than their field take the per-element kernels
            if (bits == 8) return quantize_blocks_rows<F, 8, false, kEncInt>(s, a, g, qp);
            break;
        case kEncE4M3: if (bits == 8) return quantize_blocks_rows<F, 8, false, kEncE4M3>(s, a, g, qp); break;
        case kEncE5M2: if (bits == 8) return quantize_blocks_rows<F, 8, false, kEncE5M2>(s, a, g, qp); break;
        case kEncE2M1: if (bits == 4) return quantize_blocks_rows<F, 4, false, kEncE2M1>(s, a, g, qp); break;
    }
    return hipErrorInvalidValue;
}

}  // namespace

bool blocks_dynamic_supported(int dtype, int bits, const RowArgs& a) {
    const uint32_t per_chunk = dtype == CQ_F32 ? 4 : 8;
    if (a.tensor_level) return false;
    const uint32_t bc = a.block[a.rank - 1];
    if (bc % per_chunk) return false;
    BlocksGeom g;
    return a.rows != 0 && a.shape[a.rank - 1] != 0 && blocks_geom(per_chunk, static_cast<uint32_t>(bits), a, &g);
}

hipError_t launch_quantize_blocks_dynamic(hipStream_t s, int dtype, int bits, const RowArgs& a) {
    CQ_SWITCH_DTYPE(dtype, return quantize_blocks<kF>(s, bits, a))
}

uint32_t rows_unit_values(int dtype, int bits) {
    const uint32_t per_chunk = dtype == CQ_F32 ? 4 : 8, per_word = 32u / static_cast<uint32_t>(bits);
    return per_chunk > per_word ? per_chunk : per_word;
}

hipError_t launch_quantize_rows(hipStream_t s, int dtype, int bits, const RowArgs& a) {
    if (a.rows == 0 || a.shape[a.rank - 1] == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, return quantize_rows<kF>(s, bits, a))
}

hipError_t launch_dequantize_rows(hipStream_t s, int dtype, int bits, const RowArgs& a) {
    if (a.rows == 0 || a.shape[a.rank - 1] == 0) return hipSuccess;
    CQ_SWITCH_DTYPE(dtype, return dequantize_rows<kF>(s, bits, a))
}

hipError_t launch_scales_rows(hipStream_t s, int dtype, int out_dtype, const RowArgs& args) {
    RowArgs a = args;
    const uint32_t last = a.rank - 1;
    const uint32_t per_chunk = dtype == CQ_F32 ? 4 : 8;
    const uint32_t br = a.rank >= 2 ? a.block[last - 1] : 1u;
    const uint32_t chunks_per_row = a.shape[last] / per_chunk;
    const uint32_t chunks_per_block = a.block[last] / per_chunk;
    const uint64_t block_rows = a.rows / br;
    if (block_rows == 0 || chunks_per_row == 0) return hipSuccess;
    // lanes along the row: whole blocks only, so that a block never straddles two workgroups
    a.tj_log2 = lanes_log2(chunks_per_row);
    while ((1u << a.tj_log2) < chunks_per_block) a.tj_log2++;
    if (a.tj_log2 > 8) return hipErrorInvalidValue;  // a block wider than a workgroup: not for this kernel
    const uint32_t tj_eff = ((1u << a.tj_log2) / chunks_per_block) * chunks_per_block;
    const uint32_t tr = kThreads >> a.tj_log2;
    const dim3 grid(static_cast<uint32_t>((block_rows + tr - 1) / tr), (chunks_per_row + tj_eff - 1) / tj_eff);
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((scales_rows_kernel<kF>), grid, dim3(kThreads), 0, s, a, out_dtype,
                                              static_cast<uint32_t>(block_rows), chunks_per_block, tj_eff);
                    return hipGetLastError())
}

hipError_t launch_absmax_partials_rows(hipStream_t s, int dtype, const RowArgs& args, float* partials,
                                       uint32_t* num_partials) {
    RowArgs a = args;
    const uint32_t per_chunk = dtype == CQ_F32 ? 4 : 8;
    const uint32_t chunks_per_row = a.shape[a.rank - 1] / per_chunk;
    a.tj_log2 = lanes_log2(chunks_per_row);
    const uint32_t tr = kAbsmaxThreads >> a.tj_log2;
    const uint32_t row_tiles = static_cast<uint32_t>((a.rows + tr - 1) / tr);
    const uint32_t col_tiles = (chunks_per_row + (1u << a.tj_log2) - 1) >> a.tj_log2;
    const uint64_t tiles = static_cast<uint64_t>(row_tiles) * col_tiles;
    if (tiles >= (1ull << 32)) return hipErrorInvalidValue;  // cannot happen below 2^48 elements: a tile holds 4096 of them or more
    const uint32_t grid = static_cast<uint32_t>(tiles < 1 ? 1 : (tiles > kMaxPartials ? kMaxPartials : tiles));
    *num_partials = grid;
    CQ_SWITCH_DTYPE(dtype, hipLaunchKernelGGL((absmax_rows_kernel<kF>), dim3(grid), dim3(kAbsmaxThreads), 0, s, a, partials,
                                              row_tiles, col_tiles);
                    return hipGetLastError())
}

}  // namespace cq
