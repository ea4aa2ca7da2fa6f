// Strided quantized tensor -> contiguous tensor packed along the last dimension:
// the re-packing cubek-matmul asks of cubecl-std's into_contiguous_packed before it
// hands quantized operands to its kernels (crates/cubek-matmul/src/base.rs:505-529).
// Stored element `pos` of the output gathers the logical values pos*P .. pos*P+P-1
// (P values per stored element, value 0 in the low bits); the input holds P values
// per element along `packed_dim` and is addressed through its strides.
#include "cq_device.hpp"
#include "cq_device.hpp"
#include "cq_internal.hpp"
#include "cq_magic_div.hpp"

#include <cstring>

namespace cq {
namespace {

constexpr int kThreads = 256;

// One thread per output element, any rank and strides.
template <class W>
__global__ __launch_bounds__(kThreads) void repack_generic_kernel(RepackArgs a) {
    const uint64_t pos = static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (pos >= a.num_out) return;
    const int last = static_cast<int>(a.rank) - 1;
    const W* in = static_cast<const W*>(a.input);
    // offset of the input element that holds the first of the P logical values
    uint64_t rem = pos, base = 0;
    uint32_t sub = 0;
    for (int d = last; d >= 0; d--) {
        const uint32_t n = d == last ? a.shape[d] / a.packing : a.shape[d];
        uint64_t c = rem % n;
        rem /= n;
        if (static_cast<uint32_t>(d) == a.packed_dim) {
            if (d != last) {
                sub = static_cast<uint32_t>(c % a.packing);
                c /= a.packing;
            }
        } else if (d == last) {
            c *= a.packing;
        }
        base += c * a.strides[d];
    }
    uint32_t out;
    if (static_cast<int>(a.packed_dim) == last) {
        out = in[base];  // same packing on both sides: a strided copy
    } else {
        const uint32_t mask = a.bits == 32 ? 0xffffffffu : (1u << a.bits) - 1u;
        out = 0;
        for (uint32_t k = 0; k < a.packing; k++)
            out |= ((static_cast<uint32_t>(in[base + k * a.strides[last]]) >> (sub * a.bits)) & mask) << (k * a.bits);
    }
    static_cast<W*>(a.output)[pos] = static_cast<W>(out);
}

// ---- packed along the last dimension, which is contiguous: a copy of strided rows ----
// One lane per unit of the output (16 bytes where rows, strides and pointers allow, else one stored
// element), four units in flight per lane.  The unit number, taken apart dimension by dimension
// (innermost first: the row in units, then the other dimensions; multiply-and-shift divisions), gives
// the unit's place in the input.
struct CopyLevels {
    uint32_t levels;
    uint32_t count[CQ_MAX_RANK], magic[CQ_MAX_RANK], shift[CQ_MAX_RANK];
    uint64_t in[CQ_MAX_RANK];  // input stride of the level, in units
};
template <class V>
__global__ __launch_bounds__(kThreads) void repack_rows_kernel(const V* __restrict__ in, V* __restrict__ out, CopyLevels r,
                                                               uint32_t total) {
    constexpr int kUnroll = 4;
    const uint32_t first = blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
    V v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint32_t n = first + u * kThreads;
        n = n < total ? n : total - 1;
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
        v[u] = __builtin_nontemporal_load(in + off);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint32_t n = first + u * kThreads;
        if (n < total) __builtin_nontemporal_store(v[u], out + n);
    }
}

// Fills `r` for units of `unit` stored elements and returns true when the copy kernel can take the launch.
bool plan_rows_copy(const RepackArgs& a, uint32_t unit, CopyLevels* r, uint32_t* total) {
    const uint32_t last = a.rank - 1;
    if (a.packed_dim != last || a.strides[last] != 1) return false;
    const uint64_t row = a.shape[last] / a.packing;  // stored elements per row
    if (row % unit != 0 || a.num_out / unit >= (1ull << 31)) return false;
    *r = CopyLevels{};
    const auto push = [&](uint64_t count, uint64_t stride) {
        const uint32_t k = r->levels;
        if (k > 0 && stride == r->in[k - 1] * r->count[k - 1] && r->count[k - 1] * count < (1ull << 31)) {
            r->count[k - 1] *= static_cast<uint32_t>(count);
        } else {
            r->count[k] = static_cast<uint32_t>(count);
            r->in[k] = stride;
            r->levels = k + 1;
        }
    };
    push(row / unit, 1);
    for (int d = static_cast<int>(last) - 1; d >= 0; d--) {
        if (a.shape[d] == 1) continue;
        if (a.strides[d] % unit != 0) return false;
        push(a.shape[d], a.strides[d] / unit);
    }
    for (uint32_t l = 0; l < r->levels; l++) magic_of(r->count[l], &r->magic[l], &r->shift[l]);
    *total = static_cast<uint32_t>(a.num_out / unit);
    return true;
}

// ---- tiled transposition: packed along a stride-1 dimension that is not the last ----
// In the plane of (packed dim p, last dim l) the input is [l][p / P] words and the
// output [p][l / P] words.  A block of P input words (P consecutive l, one word
// column) holds a P x P matrix of fields whose transpose is P output words (P
// consecutive p, one word column).  A workgroup moves a tile of 32*P input rows x
// 32 or 64 word columns: every thread loads four such blocks with 16-byte loads,
// transposes them in registers, scatters the words into LDS laid out as the output
// tile (word columns * P rows x 32 words), and the workgroup streams that out in 16-byte stores.
struct TileArgs {
    const uint32_t* in;
    uint32_t* out;
    uint32_t wp, wl;        // input words along p, output words along l
    uint32_t tiles_p, tiles_l;  // tiles along p and along l
    uint32_t by_xcd;            // tiles numbered XCD by XCD (launches of 2048 tiles and more)
    uint64_t in_l_stride;   // input stride of the last dimension, in words
    uint64_t out_p_stride;  // output stride of the packed dimension, in words
    uint32_t num_batch_dims;
    uint32_t batch_shape[CQ_MAX_RANK];
    uint64_t batch_in[CQ_MAX_RANK], batch_out[CQ_MAX_RANK];
};

// Transpose the kP x kP matrix of (32/kP)-bit fields held in kP words: field s of word
// i <-> field i of word s.  Recursive off-diagonal block swaps.
template <int kP>
__device__ __forceinline__ void transpose_fields(uint32_t (&a)[kP]) {
    constexpr int kBits = 32 / kP;
#pragma unroll
    for (int b = 1; b < kP; b <<= 1) {
        uint32_t mask = 0;  // fields whose index has bit `b` clear
#pragma unroll
        for (int f = 0; f < kP; f++)
            if (!(f & b)) mask |= ((kBits == 32 ? 0u : (1u << kBits)) - 1u) << (f * kBits);
#pragma unroll
        for (int r = 0; r < kP; r++) {
            if (r & b) continue;
            const uint32_t t = ((a[r] >> (b * kBits)) ^ a[r + b]) & mask;
            a[r + b] ^= t;
            a[r] ^= t << (b * kBits);
        }
    }
}

// kTileWords: input word columns per tile (a multiple of 4, at most 64);
// kTileCols: output word columns per tile (input rows / kP).
template <int kP, int kTileWords, int kTileCols>
__global__ __launch_bounds__(kTileWords / 4 * kTileCols) void repack_tile_kernel(TileArgs a) {
    constexpr int kQuads = kTileWords / 4;   // 16-byte word quads per tile row of the input
    constexpr int kT = kQuads * kTileCols;   // threads
    constexpr int kTileRows = kTileWords * kP;  // output rows (p values) per tile
    constexpr int kRot = 64 / kQuads >= 4 ? 64 / kQuads : 4;
    __shared__ uint32_t lds[kTileRows * kTileCols];
    const uint32_t pq = threadIdx.x % kQuads, lw = threadIdx.x / kQuads;
    // Workgroup i of a launch runs on XCD i % 8, each with an L2 of its own.  In launches of many tiles XCD x takes
    // the x-th eighth of the tiles, in order (along the packed dimension first, for 8-bit fields along the last
    // one), so that neighbouring tiles pass through one L2: transposed 4-bit codes [8192, 28672] 47.5 -> 45.9 us,
    // with a row pitch of 8320 words' worth 54.2 -> 48.3 us; 8-bit fields 96.6 -> 88.9 us.  The grid is
    // (8 * ceil(tiles / 8), 1, batches).
    const uint32_t per_xcd = gridDim.x / 8;
    const uint32_t tile = a.by_xcd ? (blockIdx.x % 8) * per_xcd + blockIdx.x / 8 : blockIdx.x;
    if (tile >= a.tiles_p * a.tiles_l) return;  // the whole workgroup
    const bool p_first = kP != 4 || !a.by_xcd;
    const uint32_t pw0 = (p_first ? tile % a.tiles_p : tile / a.tiles_l) * kTileWords;
    const uint32_t lw0 = (p_first ? tile / a.tiles_p : tile % a.tiles_l) * kTileCols;
    uint64_t in_base = 0, out_base = 0;
    {
        uint32_t rem = blockIdx.z;
        for (int d = static_cast<int>(a.num_batch_dims) - 1; d >= 0; d--) {
            const uint32_t c = rem % a.batch_shape[d];
            rem /= a.batch_shape[d];
            in_base += c * a.batch_in[d];
            out_base += c * a.batch_out[d];
        }
    }
    const uint32_t pw = pw0 + 4 * pq;
    if (pw < a.wp && lw0 + lw < a.wl) {
        u32x4 raw[kP];
        const uint32_t* src = a.in + in_base + static_cast<uint64_t>(lw0 + lw) * kP * a.in_l_stride + pw;
#pragma unroll
        for (int i = 0; i < kP; i++) raw[i] = stream_load(reinterpret_cast<const u32x4*>(src + i * a.in_l_stride));
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint32_t blk[kP];
#pragma unroll
            for (int i = 0; i < kP; i++) blk[i] = raw[i][q];
            transpose_fields<kP>(blk);
            // all rows start at the same bank; rotating the columns by a multiple of pq
            // spreads the lanes of a wave evenly over the banks
            const uint32_t col = (lw + pq * kRot) % kTileCols;
#pragma unroll
            for (int s = 0; s < kP; s++) lds[((4 * pq + q) * kP + s) * kTileCols + col] = blk[s];
        }
    }
    __syncthreads();
    constexpr int kRowsPerPass = kT / (kTileCols / 4);
#pragma unroll
    for (int r = 0; r < kTileRows / kRowsPerPass; r++) {
        const uint32_t row = r * kRowsPerPass + threadIdx.x / (kTileCols / 4), c4 = (threadIdx.x % (kTileCols / 4)) * 4;
        const uint64_t p = static_cast<uint64_t>(pw0) * kP + row;
        if (p < static_cast<uint64_t>(a.wp) * kP && lw0 + c4 < a.wl) {
            const uint32_t col = (c4 + (row / (4 * kP)) * kRot) % kTileCols;
            const u32x4 v = *reinterpret_cast<const u32x4*>(&lds[row * kTileCols + col]);
            stream_store(v, reinterpret_cast<u32x4*>(a.out + out_base + p * a.out_p_stride + lw0 + c4));
        }
    }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Fills `t` and returns true when the tiled kernel can take the launch.
bool plan_tiles(const RepackArgs& a, TileArgs* t, dim3* grid, uint32_t tile_words, uint32_t tile_cols) {
    const uint32_t last = a.rank - 1, pd = a.packed_dim;
    if (a.elem_bytes != 4 || (a.packing != 4 && a.packing != 8 && a.packing != 16)) return false;
    if (a.rank < 2 || pd == last || a.strides[pd] != 1) return false;
    if (!aligned16(a.input) || !aligned16(a.output)) return false;
    std::memset(t, 0, sizeof(*t));
    t->in = static_cast<const uint32_t*>(a.input);
    t->out = static_cast<uint32_t*>(a.output);
    t->wp = a.shape[pd] / a.packing;
    t->wl = a.shape[last] / a.packing;
    if (t->wp % 4 || t->wl % 4) return false;
    t->in_l_stride = a.strides[last];
    if (t->in_l_stride % 4) return false;
    // contiguous strides of the output [.., shape[last] / packing]
    uint64_t ostride[CQ_MAX_RANK], acc = 1;
    for (int d = static_cast<int>(last); d >= 0; d--) {
        ostride[d] = acc;
        acc *= static_cast<uint32_t>(d) == last ? t->wl : a.shape[d];
    }
    t->out_p_stride = ostride[pd];
    uint64_t batches = 1;
    for (uint32_t d = 0; d < a.rank; d++) {
        if (d == pd || d == last) continue;
        if (a.strides[d] % 4) return false;
        t->batch_shape[t->num_batch_dims] = a.shape[d];
        t->batch_in[t->num_batch_dims] = a.strides[d];
        t->batch_out[t->num_batch_dims] = ostride[d];
        t->num_batch_dims++;
        batches *= a.shape[d];
    }
    const uint64_t tiles_p = (t->wp + tile_words - 1) / tile_words;
    const uint64_t tiles_l = (t->wl + tile_cols - 1) / tile_cols;
    if (batches > 65535 || tiles_p * tiles_l > 0x7ffffff0ull) return false;
    t->tiles_p = static_cast<uint32_t>(tiles_p);
    t->tiles_l = static_cast<uint32_t>(tiles_l);
    t->by_xcd = tiles_p * tiles_l >= 2048;
    *grid = dim3(static_cast<uint32_t>((tiles_p * tiles_l + 7) / 8 * 8), 1, static_cast<uint32_t>(batches));
    return true;
}

// Bytes holding two 4-bit values, low nibble first, are bit for bit u32 words holding
// eight (little endian): when everything is a multiple of a word, re-express the launch
// in words so that the tiled kernel can take it.
bool bytes_as_words(const RepackArgs& a, RepackArgs* w) {
    const uint32_t last = a.rank - 1, pd = a.packed_dim;
    if (a.elem_bytes != 1 || a.packing != 2 || a.rank < 2 || pd == last || a.strides[pd] != 1) return false;
    if (a.shape[pd] % 8 || a.shape[last] % 8) return false;
    *w = a;
    w->elem_bytes = 4;
    w->packing = 8;
    w->bits = 4;
    for (uint32_t d = 0; d < a.rank; d++) {
        if (d == pd) continue;
        if (a.strides[d] % 4) return false;
        w->strides[d] = a.strides[d] / 4;
    }
    w->num_out = a.num_out / 4;
    return true;
}

}  // namespace

hipError_t launch_repack(hipStream_t s, const RepackArgs& bytes_or_words) {
    if (bytes_or_words.num_out == 0) return hipSuccess;
    RepackArgs as_words;
    const RepackArgs& a = bytes_as_words(bytes_or_words, &as_words) ? as_words : bytes_or_words;
    const RepackArgs& g = bytes_or_words;  // the per-element kernel takes the launch as it came
    TileArgs t;
    dim3 tile_grid;
    // tile = 32 output word columns x (64 | 32 | 32) input word columns for P = 4 | 8 | 16:
    // both sides move whole 128-byte lines (64-byte segments measured at two thirds of this)
    const uint32_t tile_words = a.packing == 4 ? 64 : 32;
    if (plan_tiles(a, &t, &tile_grid, tile_words, 32)) {
        switch (a.packing) {
            case 4: hipLaunchKernelGGL((repack_tile_kernel<4, 64, 32>), tile_grid, dim3(512), 0, s, t); break;
            case 8: hipLaunchKernelGGL((repack_tile_kernel<8, 32, 32>), tile_grid, dim3(256), 0, s, t); break;
            default: hipLaunchKernelGGL((repack_tile_kernel<16, 32, 32>), tile_grid, dim3(256), 0, s, t); break;
        }
        return hipGetLastError();
    }
    // the same packing on both sides: strided rows, copied in 16-byte units where everything is aligned
    CopyLevels levels;
    uint32_t total = 0;
    const uint32_t per16 = 16 / g.elem_bytes;
    if (aligned16(g.input) && aligned16(g.output) && plan_rows_copy(g, per16, &levels, &total)) {
        hipLaunchKernelGGL((repack_rows_kernel<u32x4>), dim3((total + kThreads * 4 - 1) / (kThreads * 4)), dim3(kThreads), 0, s,
                           static_cast<const u32x4*>(g.input), static_cast<u32x4*>(g.output), levels, total);
        return hipGetLastError();
    }
    if (g.elem_bytes == 4 && plan_rows_copy(g, 1, &levels, &total)) {
        hipLaunchKernelGGL((repack_rows_kernel<uint32_t>), dim3((total + kThreads * 4 - 1) / (kThreads * 4)), dim3(kThreads), 0, s,
                           static_cast<const uint32_t*>(g.input), static_cast<uint32_t*>(g.output), levels, total);
        return hipGetLastError();
    }
    const dim3 grid(static_cast<uint32_t>((g.num_out + kThreads - 1) / kThreads));
    if (g.elem_bytes == 4)
        hipLaunchKernelGGL((repack_generic_kernel<uint32_t>), grid, dim3(kThreads), 0, s, g);
    else
        hipLaunchKernelGGL((repack_generic_kernel<uint8_t>), grid, dim3(kThreads), 0, s, g);
    return hipGetLastError();
}

}  // namespace cq
