// Yardsticks for bench.py, not part of the product library: kernels that move bytes and compute nothing, launched the
// way the streaming kernels are (workgroups of 256 lanes, four 16-byte accesses per lane, consecutive lanes on
// consecutive 16 bytes).  They say what this GPU's memory gives a pure read stream, a pure write stream and a copy
// of a given size, beside the 8 TB/s of the data sheet, and serve as the copy of known size that the FETCH_SIZE /
// WRITE_SIZE counters are scaled with.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256, kUnroll = 4;

__global__ __launch_bounds__(kThreads) void probe_read_kernel(const u32x4* __restrict__ in, uint32_t* __restrict__ sink) {
    const u32x4* p = in + static_cast<uint64_t>(blockIdx.x) * kThreads * kUnroll + threadIdx.x;
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) v[u] = __builtin_nontemporal_load(p + u * kThreads);
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    if (acc == 0x9e3779b9u && sink != nullptr) sink[0] = acc;  // keeps the loads; practically never taken
}

__global__ __launch_bounds__(kThreads) void probe_write_kernel(u32x4* __restrict__ out) {
    u32x4* p = out + static_cast<uint64_t>(blockIdx.x) * kThreads * kUnroll + threadIdx.x;
    const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
#pragma unroll
    for (int u = 0; u < kUnroll; u++) __builtin_nontemporal_store(v, p + u * kThreads);
}

__global__ __launch_bounds__(kThreads) void probe_copy_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out) {
    const uint64_t at = static_cast<uint64_t>(blockIdx.x) * kThreads * kUnroll + threadIdx.x;
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) v[u] = __builtin_nontemporal_load(in + at + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) __builtin_nontemporal_store(v[u], out + at + u * kThreads);
}

// The traffic of a quantize launch without its arithmetic: a workgroup reads its 1024 chunks and writes `narrow` <= 1024
// chunks (codes and scales are that much smaller than the floats), consecutive lanes on consecutive 16 bytes on both
// sides; what it writes depends on what it read, so the loads stay.
__global__ __launch_bounds__(kThreads) void probe_narrow_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out, uint32_t narrow) {
    const uint64_t at = static_cast<uint64_t>(blockIdx.x) * kThreads * kUnroll + threadIdx.x;
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) v[u] = __builtin_nontemporal_load(in + at + u * kThreads);
    const u32x4 x = v[0] ^ v[1] ^ v[2] ^ v[3];
    u32x4* o = out + static_cast<uint64_t>(blockIdx.x) * narrow + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kUnroll; u++)
        if (u * kThreads + threadIdx.x < narrow) __builtin_nontemporal_store(x, o + u * kThreads);
}

// ... and of a dequantize launch: a workgroup reads `narrow` chunks and writes 1024.
__global__ __launch_bounds__(kThreads) void probe_widen_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out, uint32_t narrow) {
    const u32x4* p = in + static_cast<uint64_t>(blockIdx.x) * narrow + threadIdx.x;
    u32x4 x = {threadIdx.x, blockIdx.x, 3u, 4u};
#pragma unroll
    for (int u = 0; u < kUnroll; u++)
        if (u * kThreads + threadIdx.x < narrow) x ^= __builtin_nontemporal_load(p + u * kThreads);
    const uint64_t at = static_cast<uint64_t>(blockIdx.x) * kThreads * kUnroll + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) __builtin_nontemporal_store(x, out + at + u * kThreads);
}

// The traffic of the quantize (kWiden false) or dequantize (kWiden true) tile kernels for a bf16 tensor stored
// transposed, element (r, c) at c * rows + r, without the arithmetic: a workgroup moves a tile of 128 rows x 256
// columns: 256 runs of 256 bytes of floats `rows` elements apart on one side, 128 bytes of 4-bit codes and 32 bytes of
// f32 scales (blocks of 32) per row on the other.  kPlain: ordinary stores instead of streaming ones; kXcd: consecutive
// tiles on one XCD (workgroups go round the eight XCDs).
template <bool kWiden, bool kPlain, bool kXcd>
__global__ __launch_bounds__(kThreads) void probe_transposed_tile_kernel(char* __restrict__ floats, char* __restrict__ codes,
                                                                         char* __restrict__ scales, uint32_t rows, uint32_t cols) {
    const uint32_t tiles_c = cols / 256u;
    uint32_t b = blockIdx.x;
    if (kXcd) {
        const uint32_t n = gridDim.x / 8u;
        if (b < n * 8u) b = (b % 8u) * n + b / 8u;
    }
    const uint32_t tr = b / tiles_c, tc = b % tiles_c, t = threadIdx.x;
    char* fbase = floats + static_cast<uint64_t>(tc) * 256u * rows * 2u + static_cast<uint64_t>(tr) * 256u;
    const auto float_piece = [&](uint32_t p) {  // piece p of the tile: column p / 16, 16 bytes p % 16 of its run
        return reinterpret_cast<u32x4*>(fbase + static_cast<uint64_t>(p / 16u) * rows * 2u + (p % 16u) * 16u);
    };
    const auto code_piece = [&](uint32_t p) {  // row p / 8, 16 bytes p % 8 of its 128
        return reinterpret_cast<u32x4*>(codes + (static_cast<uint64_t>(tr) * 128u + p / 8u) * (cols / 2u) + static_cast<uint64_t>(tc) * 128u + (p % 8u) * 16u);
    };
    u32x4* scale_piece = reinterpret_cast<u32x4*>(scales + (static_cast<uint64_t>(tr) * 128u + t / 2u) * (cols / 8u) + static_cast<uint64_t>(tc) * 32u + (t % 2u) * 16u);
    const auto put = [](u32x4 v, u32x4* at) {
        if (kPlain) *at = v; else __builtin_nontemporal_store(v, at);
    };
    u32x4 acc = {t, b, 3u, 4u};
    if (!kWiden) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            u32x4 v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = __builtin_nontemporal_load(float_piece((s * 4 + j) * kThreads + t));
#pragma unroll
            for (int j = 0; j < 4; j++) acc ^= v[j];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) put(acc, code_piece(j * kThreads + t));
        put(acc, scale_piece);
    } else {
        u32x4 v[5];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = __builtin_nontemporal_load(code_piece(j * kThreads + t));
        v[4] = __builtin_nontemporal_load(scale_piece);
#pragma unroll
        for (int j = 0; j < 5; j++) acc ^= v[j];
#pragma unroll
        for (int j = 0; j < 16; j++) put(acc, float_piece(j * kThreads + t));
    }
}

}  // namespace

// kind 0: read `bytes` of `a`; 1: write `bytes` of `b`; 2: copy `bytes` from `a` to `b`.  `bytes` is rounded down to
// whole workgroup tiles of 16 KiB; returns the bytes a launch moves in each direction through *moved, or a negative
// value for bad arguments, or the hipError_t of the launch.
extern "C" int cq_probe_run(int kind, void* stream, const void* a, void* b, uint64_t bytes, uint32_t* sink, uint64_t* moved) {
    const uint64_t tile = static_cast<uint64_t>(kThreads) * kUnroll * 16;
    const uint64_t tiles = bytes / tile;
    if (tiles == 0 || tiles >= (1ull << 31) || kind < 0 || kind > 2) return -1;
    if (moved != nullptr) *moved = tiles * tile;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<uint32_t>(tiles)), block(kThreads);
    if (kind == 0)
        hipLaunchKernelGGL(probe_read_kernel, grid, block, 0, s, static_cast<const u32x4*>(a), sink);
    else if (kind == 1)
        hipLaunchKernelGGL(probe_write_kernel, grid, block, 0, s, static_cast<u32x4*>(b));
    else
        hipLaunchKernelGGL(probe_copy_kernel, grid, block, 0, s, static_cast<const u32x4*>(a), static_cast<u32x4*>(b));
    return static_cast<int>(hipGetLastError());
}

// A launch with the traffic of a quantize (widen == 0: reads `bytes` of `wide`, writes narrow_chunks of every 1024
// chunks of that to `narrow`) or of a dequantize (widen != 0: reads the narrow side, writes `bytes` of `wide`) launch
// and none of the arithmetic.  `bytes` is rounded down to whole tiles of 16 KiB; 1 <= narrow_chunks <= 1024; the bytes
// moved on each side come back through *moved_wide / *moved_narrow.  Returns as cq_probe_run does.
extern "C" int cq_probe_shape(int widen, void* stream, void* wide, void* narrow, uint64_t bytes, uint32_t narrow_chunks,
                              uint64_t* moved_wide, uint64_t* moved_narrow) {
    const uint64_t tile = static_cast<uint64_t>(kThreads) * kUnroll * 16;
    const uint64_t tiles = bytes / tile;
    if (tiles == 0 || tiles >= (1ull << 31) || narrow_chunks == 0 || narrow_chunks > kThreads * kUnroll) return -1;
    if (moved_wide != nullptr) *moved_wide = tiles * tile;
    if (moved_narrow != nullptr) *moved_narrow = tiles * narrow_chunks * 16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<uint32_t>(tiles)), block(kThreads);
    if (widen == 0)
        hipLaunchKernelGGL(probe_narrow_kernel, grid, block, 0, s, static_cast<const u32x4*>(wide), static_cast<u32x4*>(narrow), narrow_chunks);
    else
        hipLaunchKernelGGL(probe_widen_kernel, grid, block, 0, s, static_cast<const u32x4*>(narrow), static_cast<u32x4*>(wide), narrow_chunks);
    return static_cast<int>(hipGetLastError());
}

// The transposed tile kernels' traffic for a bf16 [rows, cols] tensor stored transposed (`floats`: rows * cols * 2
// bytes; `codes`: rows * cols / 2; `scales`: rows * cols / 8), rows a multiple of 128 and cols of 256.  widen: 0 reads
// the floats and writes codes and scales, 1 the reverse; plain_stores / xcd_order pick the variant.
extern "C" int cq_probe_transposed(int widen, int plain_stores, int xcd_order, void* stream, void* floats, void* codes,
                                   void* scales, uint32_t rows, uint32_t cols) {
    if (rows == 0 || cols == 0 || rows % 128u != 0 || cols % 256u != 0) return -1;
    const uint64_t tiles = static_cast<uint64_t>(rows / 128u) * (cols / 256u);
    if (tiles >= (1ull << 31)) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<uint32_t>(tiles)), block(kThreads);
    const int variant = (widen ? 4 : 0) | (plain_stores ? 2 : 0) | (xcd_order ? 1 : 0);
#define CQ_PROBE_TILE(W, P, X)                                                                                       \
    hipLaunchKernelGGL((probe_transposed_tile_kernel<W, P, X>), grid, block, 0, s, static_cast<char*>(floats),      \
                       static_cast<char*>(codes), static_cast<char*>(scales), rows, cols)
    switch (variant) {
        case 0: CQ_PROBE_TILE(false, false, false); break;
        case 1: CQ_PROBE_TILE(false, false, true); break;
        case 2: CQ_PROBE_TILE(false, true, false); break;
        case 3: CQ_PROBE_TILE(false, true, true); break;
        case 4: CQ_PROBE_TILE(true, false, false); break;
        case 5: CQ_PROBE_TILE(true, false, true); break;
        case 6: CQ_PROBE_TILE(true, true, false); break;
        default: CQ_PROBE_TILE(true, true, true); break;
    }
#undef CQ_PROBE_TILE
    return static_cast<int>(hipGetLastError());
}
