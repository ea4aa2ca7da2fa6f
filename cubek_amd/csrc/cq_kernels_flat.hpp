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
// quantize_flat_rows_kernel / dequantize_flat_rows_kernel run the same bodies over pitched rows
// (grid y, z = the row), each row a run of chunks of its own.
//
// HBM traffic per element is the algorithmic minimum: the input once, the
// codes once, one scale per block.  Loads and stores carry the non-temporal
// hint: nothing is re-read.
#pragma once

#include "cq_device.hpp"

namespace cq {

// Where a chunk's scale comes from.
enum ScaleSrc : int {
    kScaleDynamic = 0,     // abs-max of the block, computed here
    kScaleGivenF = 1,      // `scale_in`, typed like the input (the reference's `scale` argument)
    kScalePartials = 2,    // per tensor: `scale_in` holds the f32 abs-max partials of pass 1; this
                           // kernel (pass 2) finishes the reduction, derives the scale and quantizes
};

// kParamF32: the stored scales are f32 (the common case, resolved at compile
//            time); otherwise `param_dtype_rt` selects f16 / bf16 at run time.
// kWide    : the value range does not fit its field (E4M3 / E5M2 in 8 bits).
// kChecked : the launch may run past `chunk_end` (ragged last tile): addresses
//            are clamped and stores masked.  Full tiles use the unchecked variant.
// kEnc     : stored encoding (kEncInt for the U32 store and native i8; e4m3 / e5m2 /
//            e2m1 for the native float stores, where kBits is the stored width).
// `first_row`: false in the launches over rows (quantize_flat_rows_kernel) for rows that do not start a
// block (per tensor: every row but the first); only the scale store looks at it.
template <class F, int kBits, int kGroup, int kScaleSrc, bool kParamF32, bool kWide, int kUnroll,
          int kThreads, bool kChecked, int kEnc>
__device__ __forceinline__ void quantize_flat_body(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end,
    const QuantParams& qp, uint32_t num_partials, bool first_row) {
    constexpr bool kDynamic = kScaleSrc == kScaleDynamic;
    static_assert(kScaleSrc != kScalePartials || kGroup == 0, "partials feed the per-tensor scale only");
    constexpr int kDiv = kGroup == 0 ? 1 : kGroup;
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;  // 64, 32, 16 or 8
    const int param_dtype = kParamF32 ? static_cast<int>(CQ_F32) : param_dtype_rt;
    const auto load_scale = [&](uint64_t i) { return F::load(scale_in, i); };
    // Pass 2 of the per-tensor reduction walks the tiles last to first: pass 1 has just read the
    // tensor first to last, so what it read last is what the L2 caches still hold.  Groups of
    // eight consecutive tiles keep their places, because workgroup i runs on XCD i % 8 and tile
    // i was read there in pass 1 (each XCD has its own L2).
    uint32_t tile = blockIdx.x;
    if constexpr (kScaleSrc == kScalePartials) {
        const uint32_t whole = gridDim.x & ~7u;
        if (tile < whole) tile = (whole - 8 - (tile & ~7u)) + (tile & 7u);
    }
    const uint64_t first = chunk_begin + static_cast<uint64_t>(tile) * (kThreads * kUnroll) + threadIdx.x;

    // All kUnroll loads are issued back to back.  Checked launches let
    // out-of-range lanes re-read the last chunk instead of branching.
    u32x4 raw[kUnroll];
    float s_given[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        if (kChecked) c = c < chunk_end ? c : chunk_end - 1;
        raw[u] = stream_load(in + c);
        if constexpr (!kDynamic && kGroup != 0 && kScaleSrc != kScalePartials) s_given[u] = load_scale(c / kDiv);
    }
    if constexpr (kScaleSrc == kScalePartials) {
        // second pass of the grid reduction: every workgroup reduces the (<= a few
        // hundred) partial maxima again — max is exact, so all agree bit for bit
        const float* partials = static_cast<const float*>(scale_in);
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
    } else if constexpr (!kDynamic && kGroup == 0) {
        const float s = load_scale(0);  // one scale for the whole tensor
#pragma unroll
        for (int u = 0; u < kUnroll; u++) s_given[u] = s;
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic

#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        const bool live = !kChecked || c < chunk_end;
        float v[kN];
        F::unpack(raw[u], v);

        float s_f;
        bool tame = false;
        if constexpr (kDynamic) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));  // NaN elements drop out
            amax = group_max<kGroup>(amax);
            tame = absmax_is_tame(amax);
            const float s32 = tame ? scale_from_absmax_tame(amax, qp) : scale_from_absmax(amax, qp.width);
            s_f = F::round(s32);
        } else {
            s_f = s_given[u];
        }
        // write_scale (src/quantize.rs:83-98): FS(scale), stored by the block's first lane
        const float s_fs = round_to_dtype(param_dtype, s_f);
        const uint64_t si = kGroup == 0 ? 0 : c / kDiv;
        const bool block_start = first_row && (kGroup == 0 ? c == 0 : (c % kDiv) == 0);
        if (scale_out != nullptr && live && block_start) store_dtype(param_dtype, scale_out, si, s_fs);
        // divisor F(FS(scale)); s_f is an F value, so f32 params leave it unchanged
        float d = s_fs;
        if constexpr (!kParamF32) d = F::round(s_fs);
        if constexpr (!(kDynamic && kParamF32 && F::kDtype != CQ_F16)) tame = divisor_is_tame(d);

        float qn[kN];  // negated codes
        quantize_values_neg<F, kN>(v, d, tame, qp.lo, qp.hi, qn);
        uint32_t w[2];
        if constexpr (kEnc == kEncInt)
            pack_chunk_neg<kBits, kN, kWide>(qn, w);
        else
            encode_chunk_neg<kEnc, kN>(qn, w);

        if constexpr (kChunkBits == 64) {
            if (live) stream_store(u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(out) + c);
        } else if constexpr (kChunkBits == 32) {
            if (live) stream_store(w[0], out + c);
        } else {
            constexpr int kLanesPerWord = 32 / kChunkBits;  // 2 or 4
            const uint32_t sub = static_cast<uint32_t>(c) & (kLanesPerWord - 1);
            const uint32_t word = group_or<kLanesPerWord>(w[0] << (sub * kChunkBits));
            if (live && sub == 0) stream_store(word, out + c / kLanesPerWord);
        }
    }
}

template <class F, int kBits, int kGroup, int kScaleSrc, bool kParamF32, bool kWide, int kUnroll,
          int kThreads, bool kChecked, int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void quantize_flat_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end,
    QuantParams qp, uint32_t num_partials) {
    quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParamF32, kWide, kUnroll, kThreads, kChecked, kEnc>(
        in, out, scale_in, scale_out, param_dtype_rt, chunk_begin, chunk_end, qp, num_partials, true);
}

// Pitched rows: grid y, z = the row; a row is a run of chunks [chunk_begin, chunk_end) of its own, and
// the rows of the four tensors start `rows.*` bytes apart; blocks of rows.scale_rows rows by a lane group
// of columns share their scale (given scales only: a fused abs-max sees one row).  A kernel of its own so
// that the launches over one contiguous run carry none of this in their prologue.
struct FlatRows {
    uint32_t count;
    uint32_t scale_rows;  // rows that share a row of scales (blocks of that many rows); >= 1
    uint64_t in, out, scale_in, scale_out;
};
template <class F, int kBits, int kGroup, int kScaleSrc, bool kParamF32, bool kWide, int kUnroll,
          int kThreads, bool kChecked, int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void quantize_flat_rows_kernel(
    const u32x4* __restrict__ in, uint32_t* __restrict__ out, const void* __restrict__ scale_in,
    void* __restrict__ scale_out, int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end,
    QuantParams qp, uint32_t num_partials, FlatRows rows) {
    const uint32_t row = blockIdx.y + blockIdx.z * gridDim.y;
    if (row >= rows.count) return;
    quantize_flat_body<F, kBits, kGroup, kScaleSrc, kParamF32, kWide, kUnroll, kThreads, kChecked, kEnc>(
        reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(in) + row * rows.in),
        reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(out) + row * rows.out),
        static_cast<const char*>(scale_in) + (row / rows.scale_rows) * rows.scale_in,
        scale_out == nullptr ? nullptr : static_cast<char*>(scale_out) + (row / rows.scale_rows) * rows.scale_out,
        param_dtype_rt, chunk_begin, chunk_end, qp, num_partials, kGroup == 0 ? row == 0 : row % rows.scale_rows == 0);
}

template <class F, int kBits, int kGroup, bool kParamF32, int kUnroll, int kThreads, bool kChecked, int kEnc>
__device__ __forceinline__ void dequantize_flat_body(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params,
    int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end) {
    const int param_dtype = kParamF32 ? static_cast<int>(CQ_F32) : param_dtype_rt;
    constexpr int kN = F::kPerChunk;
    constexpr int kChunkBits = kN * kBits;
    const uint64_t first =
        chunk_begin + static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;

    uint32_t w0[kUnroll], w1[kUnroll];
    float sc[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        if (kChecked) c = c < chunk_end ? c : chunk_end - 1;  // clamp instead of branching
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
        const uint64_t si = kGroup == 0 ? 0 : c / (kGroup == 0 ? 1 : kGroup);
        sc[u] = F::round(load_dtype(param_dtype, params, si));  // Line::cast_from(scale)
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load ahead of the arithmetic
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float y[kN];
        if constexpr (kChunkBits == 64) {
            decode_fields<kEnc, kBits, 4>(w0[u], y);
            decode_fields<kEnc, kBits, 4>(w1[u], y + 4);
        } else {
            decode_fields<kEnc, kBits, kN>(w0[u], y);
        }
#pragma unroll
        for (int i = 0; i < kN; i++) y[i] = sc[u] * y[i];
        if (!kChecked || c < chunk_end) stream_store(F::pack(y), out + c);  // pack rounds to F
    }
}

template <class F, int kBits, int kGroup, bool kParamF32, int kUnroll, int kThreads, bool kChecked,
          int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void dequantize_flat_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params,
    int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end) {
    dequantize_flat_body<F, kBits, kGroup, kParamF32, kUnroll, kThreads, kChecked, kEnc>(in, out, params, param_dtype_rt,
                                                                                         chunk_begin, chunk_end);
}
template <class F, int kBits, int kGroup, bool kParamF32, int kUnroll, int kThreads, bool kChecked,
          int kEnc = kEncInt>
__global__ __launch_bounds__(kThreads) void dequantize_flat_rows_kernel(
    const uint32_t* __restrict__ in, u32x4* __restrict__ out, const void* __restrict__ params,
    int param_dtype_rt, uint64_t chunk_begin, uint64_t chunk_end, FlatRows rows) {
    const uint32_t row = blockIdx.y + blockIdx.z * gridDim.y;
    if (row >= rows.count) return;
    dequantize_flat_body<F, kBits, kGroup, kParamF32, kUnroll, kThreads, kChecked, kEnc>(
        reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(in) + row * rows.in),
        reinterpret_cast<u32x4*>(reinterpret_cast<char*>(out) + row * rows.out),
        static_cast<const char*>(params) + (row / rows.scale_rows) * rows.scale_in, param_dtype_rt, chunk_begin, chunk_end);
}

// Block abs-max -> scale typed like the input (what quantize takes as `scale`).
template <class F, int kGroup, int kUnroll, int kThreads>
__device__ __forceinline__ void scales_flat_body(const u32x4* __restrict__ in, void* __restrict__ scales,
                                                 uint64_t num_chunks, const QuantParams& qp) {
    constexpr int kN = F::kPerChunk;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
    const uint64_t last = num_chunks - 1;
    u32x4 raw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        raw[u] = stream_load(in + (c < num_chunks ? c : last));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint64_t c = first + static_cast<uint64_t>(u) * kThreads;
        float v[kN];
        F::unpack(raw[u], v);
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < kN; i++) amax = fmaxf(amax, fabsf(v[i]));
        amax = group_max<kGroup>(amax);
        const float s32 = absmax_is_tame(amax) ? scale_from_absmax_tame(amax, qp)
                                               : scale_from_absmax(amax, qp.width);
        if (c < num_chunks && (c % kGroup) == 0) F::store(scales, c / kGroup, s32);
    }
}

template <class F, int kGroup, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void scales_flat_kernel(const u32x4* __restrict__ in,
                                                               void* __restrict__ scales,
                                                               uint64_t num_chunks, QuantParams qp) {
    scales_flat_body<F, kGroup, kUnroll, kThreads>(in, scales, num_chunks, qp);
}
// pitched rows (grid y, z = the row): rows.in / rows.scale_out bytes between the rows of the two tensors
template <class F, int kGroup, int kUnroll, int kThreads>
__global__ __launch_bounds__(kThreads) void scales_flat_rows_kernel(const u32x4* __restrict__ in,
                                                                    void* __restrict__ scales,
                                                                    uint64_t num_chunks, QuantParams qp, FlatRows rows) {
    const uint32_t row = blockIdx.y + blockIdx.z * gridDim.y;
    if (row >= rows.count) return;
    scales_flat_body<F, kGroup, kUnroll, kThreads>(
        reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(in) + row * rows.in),
        static_cast<char*>(scales) + (row / rows.scale_rows) * rows.scale_out, num_chunks, qp);
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
                    raw[u] = stream_load(in + (c < num_chunks ? c : num_chunks - 1));
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
