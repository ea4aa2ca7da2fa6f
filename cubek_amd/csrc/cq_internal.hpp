// Host-side interface between the C ABI (cq_abi.hip) and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cubek_quant.h"

namespace cq {

// Scale addressing of one launch, the data of the reference's
// ScalesLayout::{PerTensor,BlockScaled} (crates/cubek-quant/src/layout/scales.rs:15-195).
struct Layout {
    uint32_t rank;                   // 0 = per-tensor
    uint32_t shape[CQ_MAX_RANK];     // unpacked element shape
    uint32_t block[CQ_MAX_RANK];     // block extents left-padded with 1
    uint64_t stride_a[CQ_MAX_RANK];  // strides (elements) of `scale` / `params`
    uint64_t stride_b[CQ_MAX_RANK];  // strides (elements) of `out_scale`
};

struct Range {
    float lo, hi;
    uint32_t unrounded = 0;  // CQ_VALUE_E2M1_OCP: the clamped quotient goes to the e2m1 cast without the integer rounding
};

// Rows that each lane finds for itself (short rows, leading dimensions with strides of their own):
// the leading dimensions innermost first, `count` entries each, and the bytes per entry in the four tensors.
// The lane-wise kernels walk at most this many levels of leading dimensions (after neighbours that every tensor
// steps through uniformly are merged): rank 5 without any merging.  Their launch arguments live in scalar
// registers, and seven levels spilled a third of them.  Deeper layouts take the row kernels.
constexpr int kMaxLaneLevels = 4;
struct LaneLevels {
    uint32_t levels;  // 0: not used
    uint32_t count[kMaxLaneLevels];
    uint64_t in[kMaxLaneLevels], out[kMaxLaneLevels], scale_in[kMaxLaneLevels], scale_out[kMaxLaneLevels];
};

// Flat fast path: contiguous tensors, scales contiguous, blocks are runs of
// `block` consecutive elements (block == 0: one scale for the whole tensor).
struct FlatArgs {
    const void* input;    // float tensor (quantize) / u32 words (dequantize)
    void* output;         // u32 words (quantize) / float tensor (dequantize)
    const void* scale_in; // quantize with given scales (typed scale_in_dtype); dequantize: params;
                          // ScaleSource::Partials: the f32 abs-max partials of pass 1
    uint32_t num_partials;
    int scale_in_dtype;   // cq_dtype of scale_in (quantize only)
    void* scale_out;      // quantize: out_scale typed as param dtype, NULL = do not write;
                          // launch_scales_flat: scales typed like the input
    uint64_t num_chunks;  // 16-byte chunks of the float tensor handled by this launch (per row when rows > 1)
    // rows > 1: the launch covers `rows` runs of num_chunks chunks, in groups of `inner_rows` (0: one group);
    // the rows of a group start *_pitch bytes apart in the four tensors, the groups *_outer bytes.  rows 0 or 1:
    // one contiguous run
    uint64_t rows, inner_rows, in_pitch, out_pitch, scale_in_pitch, scale_out_pitch;
    uint64_t in_outer, out_outer, scale_in_outer, scale_out_outer;
    LaneLevels lanes;     // lanes.levels > 0: `rows` rows of num_chunks chunks addressed lane by lane instead
    uint32_t scale_rows;  // rows > 1, given scales: blocks of this many rows share a row of scales (0 or 1: one)
    uint32_t block;       // elements per block, 0 = per-tensor.  Launches that read their scales (given, stored,
                          // dequantize) take any whole number of 16-byte chunks, lane by lane where that number is
                          // not a power of two up to 32; a fused abs-max takes the powers of two
    int param_dtype;      // cq_dtype of the stored scales
    int encoding;         // 0 two's-complement fields (U32 store, native i8); 1 e4m3, 2 e5m2 bytes; 3 e2m1 nibbles
    Range range;
    uint32_t whole_grid = 0;  // set between the launchers' objects only: whole tiles of the run to launch
    uint32_t any_group = 0;   // set by the launchers: chunks per block where the lane-wise kernels divide by it (see `block`)
    bool lanes_only = false;  // set by the launchers: no whole-tile kernel exists for this launch (fields that wrap)
};

enum class ScaleSource { Given, Dynamic, Partials, Stored };  // Stored: lane-wise launches only (FlatArgs::lanes)

// every launcher returns hipGetLastError() of its launch
hipError_t launch_quantize_flat(hipStream_t s, int dtype, int bits, ScaleSource src, const FlatArgs& a);
hipError_t launch_dequantize_flat(hipStream_t s, int dtype, int bits, const FlatArgs& a);
hipError_t launch_scales_flat(hipStream_t s, int dtype, const FlatArgs& a);  // block abs-max -> scales typed like input
bool flat_block_supported(int dtype, uint32_t block);
// any whole number of 16-byte chunks: what the flat launches that read their scales take
bool flat_block_supported_with_scales(int dtype, uint32_t block);
// the cq_kernel_family a flat launch with these arguments runs on (whole tiles of a run, whole steps of
// pitched rows, or lane by lane)
uint32_t flat_family(const FlatArgs& a, int f_dtype);

// Per-tensor abs-max, pass 1: writes `*num_partials` f32 partial maxima.
constexpr uint32_t kMaxPartials = 256;
hipError_t launch_absmax_partials(hipStream_t s, int dtype, const void* input, uint64_t num_elems,
                                  float* partials, uint32_t* num_partials);
// Per-tensor scale from the partials: out_dtype(f_dtype(2*absmax/(hi-lo))) stored at out[0].
hipError_t launch_tensor_scale(hipStream_t s, int f_dtype, int out_dtype, const float* partials,
                               uint32_t num_partials, Range range, void* out);

// Addressing of the two value tensors of a launch when they are not contiguous
// row-major (the reference reads and writes them through linear views built from
// shape and strides: crates/cubek-quant/src/quantize.rs:309-317, src/dequantize.rs:261-270).
struct ValueStrides {
    uint32_t on;                   // 0: both contiguous, offsets are the logical indices
    uint32_t rank;
    uint32_t shape[CQ_MAX_RANK];   // unpacked element shape
    uint64_t floats[CQ_MAX_RANK];  // strides (elements) of the float tensor
    uint64_t stored[CQ_MAX_RANK];  // strides (stored elements) of the quantized tensor
};

// Generic path: any rank, any strides, N-D blocks, strided scales; one thread per stored word.
struct GenericArgs {
    const void* input;
    void* output;
    const void* scale_in;
    int scale_in_dtype;     // cq_dtype of scale_in (quantize); dequantize reads param_dtype
    void* scale_out;        // NULL = do not write out_scale
    uint64_t word_begin, word_end;  // packed words (U32 store) or stored bytes (native store)
    int param_dtype;
    int value;  // cq_value
    Range range;
    Layout layout;
    ValueStrides vs;
};
hipError_t launch_quantize_generic(hipStream_t s, int dtype, int bits, const GenericArgs& a);
hipError_t launch_dequantize_generic(hipStream_t s, int dtype, int bits, const GenericArgs& a);
// one thread per block: abs-max over the N-D block box; stores
// out_dtype(dtype(2*absmax/(hi-lo))) through layout.stride_b into scale_out
hipError_t launch_scales_generic(hipStream_t s, int dtype, int out_dtype, const GenericArgs& a,
                                 uint64_t num_blocks);
// per-tensor abs-max partials of a strided float tensor (`a.vs`, `a.input`); same
// contract as launch_absmax_partials
hipError_t launch_absmax_partials_strided(hipStream_t s, int dtype, const GenericArgs& a, uint64_t num_elems,
                                          float* partials, uint32_t* num_partials);
// native store (i8 / e4m3 / e5m2 / e2m1x2), one thread per stored byte
hipError_t launch_quantize_native(hipStream_t s, int dtype, const GenericArgs& a);
hipError_t launch_dequantize_native(hipStream_t s, int dtype, const GenericArgs& a);

// Abs-max along one axis (cq_reduce_max_abs).
struct ReduceArgs {
    const void* input;
    void* output;
    void* workspace;         // f32 partials, may be NULL
    size_t workspace_bytes;
    uint32_t rank, axis;
    uint64_t shape[CQ_MAX_RANK];
    uint64_t in_strides[CQ_MAX_RANK], out_strides[CQ_MAX_RANK];
    bool contiguous;         // input and output are contiguous row-major
    bool in_contiguous;      // the input is
    bool out_contiguous;     // the output is
    uint64_t outer, len, inner;  // the contiguous view [outer, len, inner] around the axis
};
hipError_t launch_reduce_max_abs(hipStream_t s, int dtype, const ReduceArgs& a);
uint64_t reduce_workspace_bytes(uint64_t outer, uint64_t len, uint64_t inner, int dtype);


// Row kernels: any layout whose last dimension is contiguous in both value tensors
// (N-D blocks, odd block sizes, strided scales, pitched / sliced / permuted rows).
struct RowArgs {
    const void* input;       // floats (quantize, scales) / stored words (dequantize)
    void* output;
    const void* scale_in;    // quantize: typed scale_in_dtype; dequantize: typed param_dtype
    void* scale_out;         // quantize: out_scale or NULL; scales: destination
    int scale_in_dtype, param_dtype;
    int encoding;            // cq::Encoding of the stored values
    Range range;
    uint32_t rank;
    uint32_t tensor_level;   // 1: one scale for the whole tensor
    uint32_t shape[CQ_MAX_RANK];    // unpacked shape
    uint32_t block[CQ_MAX_RANK];    // block extents left-padded with 1 (block level only)
    uint64_t fstride[CQ_MAX_RANK];  // float tensor, elements; leading strides are multiples of a 16-byte chunk
    uint64_t vstride[CQ_MAX_RANK];  // stored tensor, in 32-bit words
    uint64_t sa[CQ_MAX_RANK], sb[CQ_MAX_RANK];  // strides of scale_in / scale_out
    uint64_t rows;           // product of the leading dimensions (< 2^31)
    int32_t bc_shift;        // log2(block[last]) if a power of two, else -1
    uint32_t units_per_row, tj_log2;  // filled by the launchers
};
// values per unit of the row kernels: the last dimension and the last block extent must be multiples of it
uint32_t rows_unit_values(int dtype, int bits);
hipError_t launch_quantize_rows(hipStream_t s, int dtype, int bits, const RowArgs& a);
hipError_t launch_dequantize_rows(hipStream_t s, int dtype, int bits, const RowArgs& a);
// block abs-max -> out_dtype(dtype(2*absmax/(hi-lo))) through `sb` into scale_out; blocks may
// extend over the last two dimensions only, the last extent is a multiple of a chunk
hipError_t launch_scales_rows(hipStream_t s, int dtype, int out_dtype, const RowArgs& a);
// fused abs-max + scale + quantize for blocks over the last two dimensions whose last extent is a
// whole number of 16-byte chunks; writes scale_out (typed param_dtype), reads no scale_in
bool blocks_dynamic_supported(int dtype, int bits, const RowArgs& a);
hipError_t launch_quantize_blocks_dynamic(hipStream_t s, int dtype, int bits, const RowArgs& a);
// per-tensor abs-max partials (same contract as launch_absmax_partials)
hipError_t launch_absmax_partials_rows(hipStream_t s, int dtype, const RowArgs& a, float* partials,
                                       uint32_t* num_partials);

// Streaming kernels that stage values or scales through LDS (cq_kernels_staged.hip).
//
// Pieces: one contiguous run of blocks whose extent is not a power-of-two number of lanes (24, 40, 48 ... values).
// A block is `per` << group_log2 chunks of 16 bytes: 2^group_log2 neighbouring lanes hold it, `per` (odd) chunks each.
struct PiecesArgs {
    const void* input;     // floats
    void* output;          // stored words
    const void* scale_in;  // given scales, typed like the input (NULL: the block abs-max is computed in the launch)
    void* scale_out;       // out_scale typed param_dtype (may be NULL with given scales)
    int param_dtype, encoding;
    Range range;
    uint64_t num_chunks;   // 16-byte chunks of the run: a whole number of blocks
    uint32_t per, group_log2;
};
bool pieces_supported(int dtype, int bits, uint32_t block, uint32_t* per, uint32_t* group_log2);
hipError_t launch_quantize_pieces(hipStream_t s, int dtype, int bits, const PiecesArgs& a);

// Scale tiles: rows of 16-byte chunks (one uniform pitch per tensor) with 1-D blocks of a power-of-two number of
// lanes, whose scale tensors have any two strides (stored column by column, with a column stride, ...).  A
// workgroup takes 16 rows x 64 chunks and moves the tile's scales through LDS, so that the accesses to a scale
// tensor run along whichever of its two dimensions is closer in memory.
struct ScaleTileArgs {
    const void* input;     // floats (quantize) / stored words (dequantize)
    void* output;
    const void* scale_in;  // quantize: given scales typed scale_in_dtype, or NULL (abs-max in the launch); dequantize: params
    void* scale_out;       // quantize: out_scale typed param_dtype, or NULL
    int scale_in_dtype, param_dtype, encoding;
    Range range;
    uint32_t rows, row_chunks;          // rows of the launch, 16-byte chunks of floats per row
    uint32_t group_log2;                // lanes per block, 2^0 .. 2^5
    uint64_t float_pitch, stored_pitch; // bytes from row to row
    uint64_t stored_col;                // stored elements from one to the next along the last dimension; other than 1
                                        // (words of the U32 store only): the codes of a tile pass through LDS too
    uint64_t sa_row, sa_col, sb_row, sb_col;  // strides (elements) of scale_in / scale_out along rows and block columns
};
hipError_t launch_quantize_scale_tiles(hipStream_t s, int dtype, int bits, const ScaleTileArgs& a);
hipError_t launch_dequantize_scale_tiles(hipStream_t s, int dtype, int bits, const ScaleTileArgs& a);

// Transposed float tensors: the memory-fastest dimension is the second to last logical one.
// Blocks run along the last dimension only (or one scale per tensor).
struct TransposedArgs {
    const void* input;       // floats (quantize) / stored words (dequantize)
    void* output;
    const void* scale_in;    // quantize with given scales: typed scale_in_dtype; dequantize: typed param_dtype
    void* scale_out;         // quantize: out_scale or NULL
    int scale_in_dtype, param_dtype;
    int encoding;            // cq::Encoding
    Range range;
    uint32_t tensor_level;
    uint32_t rows;           // extent of the second to last dimension (float stride 1)
    uint32_t segment;        // columns one thread handles: the block size, or 32 per tensor
    uint32_t segments;       // last dimension / segment
    uint32_t batches;        // product of the leading dimensions (<= 65535)
    uint64_t pitch_f;        // float stride of the last dimension
    uint64_t vrow;           // stored stride of the second to last dimension, in 32-bit words
    uint64_t sa_row, sa_col, sb_row, sb_col;  // scale strides along the two dimensions
    uint32_t num_batch_dims;
    uint32_t staged;         // quads kernel, set by its launcher: 1 words, 2 scales leave through LDS as whole runs
    uint32_t batch_shape[CQ_MAX_RANK];
    uint64_t batch_f[CQ_MAX_RANK], batch_v[CQ_MAX_RANK], batch_sa[CQ_MAX_RANK], batch_sb[CQ_MAX_RANK];
};
hipError_t launch_quantize_transposed(hipStream_t s, int dtype, int bits, bool dynamic, const TransposedArgs& a);
hipError_t launch_dequantize_transposed(hipStream_t s, int dtype, int bits, const TransposedArgs& a);
// block abs-max -> out_dtype(dtype(2*absmax/(hi-lo))) through sb_row / sb_col into scale_out (block level only)
hipError_t launch_scales_transposed(hipStream_t s, int dtype, int out_dtype, const TransposedArgs& a);

// Re-packing of a strided quantized tensor (cq_into_contiguous_packed).
struct RepackArgs {
    const void* input;
    void* output;
    uint32_t elem_bytes;          // 4 (u32 words) or 1 (bytes)
    uint32_t packing, bits;       // values per stored element, bits per value
    uint32_t rank, packed_dim;
    uint32_t shape[CQ_MAX_RANK];  // logical (unpacked) shape
    uint64_t strides[CQ_MAX_RANK];  // input strides, in stored elements
    uint64_t num_out;             // stored elements of the output
};
hipError_t launch_repack(hipStream_t s, const RepackArgs& a);

// y = dequantize(W) * x over a packed [rows, cols] weight matrix (cq_gemv_quantized).
struct GemvArgs {
    const void* words;   // u32 words, row r at words + r * word_pitch
    const void* scales;  // typed param_dtype
    const void* x;       // [cols], typed dtype
    void* y;             // [rows], typed y_dtype
    int dtype, y_dtype, param_dtype;
    uint32_t bits;       // bits per value
    uint32_t native;     // 0: fields of the U32 store (and i8 bytes); 1 e4m3, 2 e5m2, 3 e2m1x2 of the native store
    uint32_t rows, cols;
    uint64_t word_pitch;
    uint32_t block_rows, block_cols;  // 0, 0: one scale per tensor
    uint64_t scale_stride_row, scale_stride_col;
    uint32_t vectors;             // right-hand vectors: x is `vectors` rows of x_stride elements, y of y_stride
    uint64_t x_stride, y_stride;
    bool x_aligned16, words_aligned16;
};
bool gemv_streams(const GemvArgs& a);  // the launch takes the streaming kernel
uint32_t gemv_vectors_per_launch(const GemvArgs& a, uint32_t remaining);
hipError_t gemv_stream_f32_scales(hipStream_t s, const GemvArgs& a);    // the streaming kernels, by object
hipError_t gemv_stream_16bit_scales(hipStream_t s, const GemvArgs& a);
hipError_t gemv_stream_batched(hipStream_t s, const GemvArgs& a);
hipError_t gemv_stream_f32_x(hipStream_t s, const GemvArgs& a);
bool gemv_mfma_takes(const GemvArgs& a);  // ... on the matrix cores (4-bit fields, blocks of 32, f32 scales, 1 - 4 vectors)
hipError_t gemv_mfma(hipStream_t s, const GemvArgs& a);
hipError_t launch_gemv_quantized(hipStream_t s, const GemvArgs& a);

}  // namespace cq
