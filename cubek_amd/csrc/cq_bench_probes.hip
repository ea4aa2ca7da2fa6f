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
