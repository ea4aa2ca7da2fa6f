/*
 * cubek_quant.h — C ABI of the MI355X (gfx950) quantize / dequantize library.
 *
 * Every entry point is what a foreign-function binding of the reference crate
 * `cubek-quant` would bind for its quantize/dequantize path.  The reference
 * interface each one replaces is cited next to it (paths are relative to the
 * reference tree, crates/cubek-quant/...).
 *
 * Conventions
 *   - plain pointers and sizes only; `ptr` fields are DEVICE pointers;
 *   - the caller owns every buffer (inputs, outputs, scales, workspace);
 *   - calls are asynchronous and ordered on the given HIP stream (NULL = the
 *     default stream); nothing here synchronises the device;
 *   - every function returns a cq_status (0 = success) and never aborts;
 *   - an entry point that launches kernels first clears the calling thread's pending HIP error
 *     (hipGetLastError), so that CQ_ERR_HIP always speaks of this call's own launches;
 *   - special values follow IEEE arithmetic on the reference's formula with these choices, which the
 *     reference leaves to its JIT backend and its tests do not observe: round() is round-half-to-even,
 *     clamp() is max(lo, min(x, hi)) with minNum/maxNum, so a NaN quotient (NaN element, NaN scale, 0/0)
 *     quantizes to q_max; abs-max ignores NaN elements; a zero result keeps the sign IEEE gives it;
 *   - calls are re-entrant and thread safe.  The library's state is the per-thread code behind
 *     cq_last_hip_error() and, for cq_quantize_dynamic_static only, one scratch array per GPU inside the
 *     library's device code, shared by all calls of that entry point on that GPU (see there).
 */
#ifndef CUBEK_QUANT_H
#define CUBEK_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CQ_ABI_VERSION 1
#define CQ_MAX_RANK 8       /* tensors of rank 1..8                               */
#define CQ_MAX_BLOCK_DIMS 5 /* same bound as the reference's BlockSize storage    */

/* Status codes. Conditions the reference answers with panic!/assert! are
 * reported as distinct codes instead (src/quantize.rs:203-206,218,273,324;
 * src/lib.rs:28-31); launch failures map to CQ_ERR_HIP (LaunchError). */
typedef enum cq_status {
    CQ_OK = 0,
    CQ_ERR_INVALID_ARGUMENT = 1,    /* NULL pointer, bad rank, bad enum value            */
    CQ_ERR_UNSUPPORTED_SCHEME = 2,  /* value/store/param combination not implemented     */
    CQ_ERR_BLOCK_NOT_DIVISIBLE = 3, /* check_block_size_compat failed (src/lib.rs:20-33) */
    CQ_ERR_SHAPE_MISMATCH = 4,      /* packed/unpacked/scales shapes do not agree        */
    CQ_ERR_NON_CONTIGUOUS = 5,      /* an output that must be contiguous row-major is not */
    CQ_ERR_WORKSPACE_TOO_SMALL = 6,
    CQ_ERR_HIP = 7,                 /* a HIP runtime call failed; see cq_last_hip_error  */
    CQ_ERR_TOO_LARGE = 8,           /* more elements than an entry point accepts         */
    CQ_ERR_INVALID_AXIS = 9,        /* reduction axis >= rank (ReduceError::InvalidAxis) */
    CQ_ERR_SCRATCH_TOO_SMALL = 10   /* cq_quantize_dynamic_static: the call needs more than CQ_STATIC_SCRATCH_BYTES */
} cq_status;

/* Float element types of value tensors and scale parameters
 * (the reference passes ElemType / StorageType: src/quantize.rs:181,
 * src/dequantize.rs:177). */
typedef enum cq_dtype {
    CQ_F32 = 0,
    CQ_F16 = 1,
    CQ_BF16 = 2
} cq_dtype;

/* QuantValue (re-exported at src/lib.rs:14). Integer ranges used by the
 * kernels: Q8F [-128,127], Q8S [-127,127], Q4F [-8,7], Q4S [-7,7],
 * Q2F [-2,1], Q2S [-1,1], E2M1 [-6,6], E4M3 [-448,448], E5M2 [-57344,57344]. */
typedef enum cq_value {
    CQ_VALUE_Q8F = 0,
    CQ_VALUE_Q8S = 1,
    CQ_VALUE_Q4F = 2,
    CQ_VALUE_Q4S = 3,
    CQ_VALUE_Q2F = 4,
    CQ_VALUE_Q2S = 5,
    CQ_VALUE_E2M1 = 6,
    CQ_VALUE_E4M3 = 7,
    CQ_VALUE_E5M2 = 8,
    /* Extension with no counterpart in the reference (never produced by, and never to be passed as, E2M1):
     * OCP microscaling FP4.  The quotient x / scale is clamped to [-6, 6] in the tensor's float type and
     * rounded ONCE, to the nearest of {0, 0.5, 1, 1.5, 2, 3, 4, 6} (ties to the even code), without the
     * integer rounding the reference applies first (src/quantize.rs:33-43), so 0.5 and 1.5 occur.  Both stores
     * hold e2m1 nibbles: eight per u32 word, value i in bits [4i, 4i+4), or two per byte, value 2k in the low
     * nibble; the two layouts are the same bytes.  Dequantize decodes the nibble and multiplies by the scale.
     * The scale rule is the common one: 2 * absmax / (6 - -6) = absmax / 6. */
    CQ_VALUE_E2M1_OCP = 9
} cq_value;

typedef enum cq_param { /* QuantParam: dtype of the stored scales */
    CQ_PARAM_F32 = 0,
    CQ_PARAM_F16 = 1,
    CQ_PARAM_BF16 = 2
} cq_param;

typedef enum cq_store { /* QuantStore */
    CQ_STORE_U32 = 0,   /* 32/size_bits codes per u32 word, element 0 in the low bits */
    CQ_STORE_NATIVE = 1 /* i8 / fp8 bytes, or two e2m1 nibbles per byte               */
} cq_store;

typedef enum cq_level { /* QuantLevel */
    CQ_LEVEL_TENSOR = 0,
    CQ_LEVEL_BLOCK = 1
} cq_level;

typedef enum cq_mode { /* QuantMode */
    CQ_MODE_SYMMETRIC = 0
} cq_mode;

/* QuantScheme.  `block` holds the block size per trailing dimension exactly as
 * the reference's QuantLevel::block([..]) does (u8 entries, at most 5); it is
 * left-padded with 1s up to the tensor rank (src/layout/scales.rs:239). */
typedef struct cq_scheme {
    uint8_t value;      /* cq_value */
    uint8_t param;      /* cq_param */
    uint8_t store;      /* cq_store */
    uint8_t level;      /* cq_level */
    uint8_t mode;       /* cq_mode  */
    uint8_t block_rank; /* number of valid entries in block[] (0 for per-tensor) */
    uint8_t block[CQ_MAX_BLOCK_DIMS];
    uint8_t reserved;   /* must be 0 */
} cq_scheme;

/* Borrowed tensor handle = the fields of the reference's TensorHandleRef
 * (handle, shape, strides, elem_size).  Strides are in elements. */
typedef struct cq_tensor {
    void* ptr;
    const uint64_t* shape;
    const uint64_t* strides;
    uint32_t rank;
    uint32_t elem_size; /* bytes per element */
} cq_tensor;

typedef struct ihipStream_t* cq_stream_t; /* == hipStream_t */

/* ---- scheme helpers (QuantScheme / QuantValue methods used by the path) ---- */

/* QuantValue::size_bits (call sites src/quantize.rs:62, src/dequantize.rs:91). */
uint32_t cq_value_size_bits(uint8_t value);
/* QuantScheme::num_quants = stored bits / value bits
 * (call sites src/quantize.rs:144,290; src/dequantize.rs:67,248). */
uint32_t cq_scheme_num_quants(const cq_scheme* scheme);
/* QuantValue::range (call sites src/quantize.rs:243,296). */
cq_status cq_value_range(uint8_t value, float* range_min, float* range_max);

/* ---- the path ---- */

/* Replaces cubek_quant::quantize::launch_ref (src/quantize.rs:174-221).
 *   input      : float tensor of dtype `input_dtype`, any strides (fastest when
 *                contiguous row-major; a contiguous last dimension is the next best)
 *   output     : U32 store -> u32 tensor, shape = input shape with the last
 *                dimension divided by num_quants (tests/suite/symmetric.rs:68-69);
 *                NATIVE store -> 1-byte tensor (E2M1: last dimension / 2);
 *                any strides that do not make two stored elements overlap
 *   scale      : scales typed as `input_dtype`, shape [1] (per-tensor) or one
 *                entry per block; its strides are honoured
 *   out_scale  : same shape as `scale`, typed as scheme->param; receives the
 *                scale of every block */
cq_status cq_quantize(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                      const cq_tensor* scale, const cq_tensor* out_scale,
                      const cq_scheme* scheme, cq_dtype input_dtype);

/* Replaces cubek_quant::dequantize::launch_ref (src/dequantize.rs:171-229).
 *   values : quantized tensor as written by cq_quantize, any strides
 *   output : float tensor of dtype `output_dtype`, unpacked shape, any strides
 *   params : scales typed as scheme->param */
cq_status cq_dequantize(cq_stream_t stream, const cq_tensor* values, const cq_tensor* output,
                        const cq_tensor* params, const cq_scheme* scheme,
                        cq_dtype output_dtype);

/* Scale production.  The reference crate leaves this to its caller; the rule is
 * the one its tests apply on the host, scale = 2*max|x| / (q_max - q_min) in f32
 * (tests/suite/symmetric.rs:35-38,156-179), with NaN elements ignored.
 *   scales : typed as `input_dtype` (what cq_quantize expects as `scale`),
 *            contiguous, shape [1] or one entry per block
 *   workspace : cq_workspace_bytes() bytes of device memory, 256-byte aligned;
 *               only per-tensor schemes use it, may be NULL for block schemes */
cq_status cq_compute_scales(cq_stream_t stream, const cq_tensor* input, const cq_tensor* scales,
                            const cq_scheme* scheme, cq_dtype input_dtype,
                            void* workspace, size_t workspace_bytes);

/* Fused abs-max + scale + quantize: same results as cq_compute_scales followed
 * by cq_quantize, without materialising the input-typed scales. */
cq_status cq_quantize_dynamic(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                              const cq_tensor* out_scale, const cq_scheme* scheme,
                              cq_dtype input_dtype, void* workspace, size_t workspace_bytes);

/* Device bytes the two entry points above need for `num_elements` inputs. */
size_t cq_workspace_bytes(const cq_scheme* scheme, uint64_t num_elements);

/* cq_quantize_dynamic without a workspace argument.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory for a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  Same arguments otherwise, same codes and
 * scales bit for bit.  The scratch memory (the abs-max partials of the per-tensor grid reduction)
 * is an array of CQ_STATIC_SCRATCH_BYTES inside the library's device code; every GPU the library
 * runs on holds its copy until the process ends.  The call allocates and frees nothing.
 *   - a call whose scheme and size need more scratch than the array holds returns
 *     CQ_ERR_SCRATCH_TOO_SMALL (cq_workspace_bytes() tells the need; today no scheme exceeds it);
 *   - the device that is current when the call is made must be the stream's device: a stream of
 *     another device returns CQ_ERR_INVALID_ARGUMENT (the array's address is per device); the first
 *     call on a device looks the array's address up and must not run under stream capture;
 *   - all calls on one GPU share that GPU's array: two calls that overlap in time on one GPU
 *     (different streams, or threads) race on it.  Calls on one stream do not overlap. */
#define CQ_STATIC_SCRATCH_BYTES 1024
cq_status cq_quantize_dynamic_static(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                                     const cq_tensor* out_scale, const cq_scheme* scheme,
                                     cq_dtype input_dtype);

/* ---- abs-max along an axis (the step in front of the path) ---- */

/* Replaces cubek_reduce::reduce::<R, MaxAbs> (crates/cubek-reduce/src/lib.rs:93-131 with
 * src/instructions/maxabs.rs:10-96), the reduction a caller runs to obtain per-row /
 * per-channel abs-max values before dividing them into scales.
 *   input  : float tensor of dtype `dtype`, any strides
 *   output : same dtype, same shape except extent 1 on `axis`
 *            (anything else: CQ_ERR_SHAPE_MISMATCH, ReduceError::MismatchShape)
 *   workspace : optional device scratch of cq_reduce_workspace_bytes() bytes (16-byte aligned); lets
 *            reductions with few outputs spread one output over many workgroups, and gives an
 *            output tensor that is not contiguous the streaming kernels too (they leave a
 *            contiguous result in the workspace, which one more small launch puts in place)
 * NaN elements are ignored; an axis of extent 0 yields 0. */
cq_status cq_reduce_max_abs(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                            uint32_t axis, cq_dtype dtype, void* workspace, size_t workspace_bytes);
size_t cq_reduce_workspace_bytes(const cq_tensor* input, uint32_t axis, cq_dtype dtype);

/* ---- re-packing of strided quantized tensors (the step behind the path) ---- */

/* Replaces cubecl_std::tensor::into_contiguous_packed as cubek-matmul calls it on a
 * quantized operand (crates/cubek-matmul/src/base.rs:505-529): a quantized tensor with
 * any strides (e.g. a transposed view) becomes a contiguous one packed along the last
 * dimension of the logical shape.
 *   input   : u32 (elem_size 4) or u8 (elem_size 1) tensor holding `packing` values per
 *             element, value 0 in the low bits, packed along the rightmost dimension
 *             whose stride is 1 (the last one if there is none); its shape is `shape`
 *             with that dimension divided by `packing`
 *   shape   : logical (unpacked) shape, `rank` entries; the last dimension and the
 *             packed dimension must be multiples of `packing`
 *   output  : contiguous, same element type, `shape` with the last dimension / packing */
cq_status cq_into_contiguous_packed(cq_stream_t stream, const cq_tensor* input, const cq_tensor* output,
                                    const uint64_t* shape, uint32_t rank, uint32_t packing);

/* ---- a consumer of the packed format (the weight-load path) ---- */

/* y = dequantize(W) * x with W read once in its quantized form: stands where the reference's matmul
 * takes a quantized operand and dequantizes it while loading (MatmulInputHandle::Quantized,
 * crates/cubek-matmul/src/base.rs:309-317; scale lookup per (row, col),
 * crates/cubek-matmul/src/components/global/memory/layout.rs:371-455), for the matrix-vector case.
 * The kernels are written against include/cubek_quant_device.hpp only.
 *   values : U32-store tensor [rows, cols / num_quants] of words, or native-store tensor of bytes ([rows, cols]
 *            for i8 / e4m3 / e5m2, [rows, cols / 2] for e2m1 pairs); rows may be pitched (stride 1 along the row)
 *   params : scales typed scheme->param, shape [1] (per tensor) or [rows / block_rows, cols / block_cols]
 *            for blocks over the last one or two dimensions, any strides
 *   x      : [cols] of `dtype`, contiguous, or [vectors, cols] with contiguous rows: as many right-hand sides
 *   y      : [rows] of `y_dtype`, contiguous, or [vectors, rows] with contiguous rows
 * Every weight enters as the value cq_dequantize would produce for `dtype`, F(F(scale) * F(code)); the
 * products are accumulated in f32 (order unspecified) and the sum is rounded once to `y_dtype`.
 * A streaming kernel (HBM- or arithmetic-bound, 45 - 70 % of the HBM peak on large weights) takes a 16-bit
 * `dtype` (f32 as well where the scales are f32) with 16-byte aligned rows of codes and x, scales of any type per tensor or on
 * blocks of 1, 2, 4, ... times 16 bytes of codes along the row (any number of rows): cq_plan_kind(CQ_OP_GEMV)
 * tells.  Four right-hand sides go through it at once (all but 2-bit fields; rows of x on 16-byte
 * boundaries), so that the weights are read and dequantized once for the four; more, or others, are
 * computed in turns.  Every other U32-store layout takes a simple
 * wave-per-row kernel; every other native-store layout is CQ_ERR_UNSUPPORTED_SCHEME. */
cq_status cq_gemv_quantized(cq_stream_t stream, const cq_tensor* values, const cq_tensor* params,
                            const cq_scheme* scheme, const cq_tensor* x, const cq_tensor* y,
                            cq_dtype dtype, cq_dtype y_dtype);

/* ---- which kernels a call would run on ---- */

/* No counterpart in the reference (its one kernel per entry point takes every layout at the same, low,
 * speed).  Here the layout of the tensors decides between kernel families whose throughput differs by more
 * than a factor of ten; this query tells a caller which one a call would take, without launching anything,
 * so that a slow path does not go unnoticed. */
typedef enum cq_kernel_family {
    CQ_FAMILY_NONE = 0,        /* nothing to launch (empty tensor)                                            */
    CQ_FAMILY_FLAT = 1,        /* contiguous tensors, whole 16 KiB tiles: the streaming kernels (HBM rate)     */
    CQ_FAMILY_FLAT_ROWS = 2,   /* the same kernels over pitched rows of whole 4 KiB steps                      */
    CQ_FAMILY_FLAT_LANES = 3,  /* the same arithmetic, every lane finding its own row: short, ragged or
                                  permuted rows, f16 / bf16 parameters, small tensors (55 - 80 % of HBM rate)  */
    CQ_FAMILY_ROWS = 4,        /* contiguous last dimension, any blocks and strides (35 - 70 %)                */
    CQ_FAMILY_BLOCKS = 5,      /* fused abs-max + quantize for blocks over the last two dimensions (55 - 70 %) */
    CQ_FAMILY_TRANSPOSED = 6,  /* float tensor whose contiguous dimension is the second to last (45 - 70 %)    */
    CQ_FAMILY_PER_ELEMENT = 7, /* everything else, one thread per stored element (3 - 30 %)                    */
    CQ_FAMILY_STAGED = 8       /* streaming kernels with one trip through LDS: fused abs-max over blocks that are
                                  not a power-of-two number of lanes (24, 40, 48 values), scale tensors stored along
                                  another dimension than the last                                              */
} cq_kernel_family;

typedef enum cq_op {
    CQ_OP_QUANTIZE = 0,          /* cq_quantize: scale and out_scale given                    */
    CQ_OP_QUANTIZE_DYNAMIC = 1,  /* cq_quantize_dynamic: `scale` ignored (may be NULL)        */
    CQ_OP_DEQUANTIZE = 2,        /* cq_dequantize: `scale` = params, `out_scale` ignored      */
    CQ_OP_COMPUTE_SCALES = 3,    /* cq_compute_scales: `values` and `out_scale` ignored       */
    CQ_OP_GEMV = 4               /* cq_gemv_quantized: `floats` = x, `scale` = params, `out_scale` = y (typed `dtype`
                                    or f32): CQ_FAMILY_FLAT for its streaming kernel, CQ_FAMILY_ROWS for the
                                    general one (a wave per row, about a third of the rate)  */
} cq_op;

/* The family of the kernel that would move the value tensors of the call (for CQ_OP_COMPUTE_SCALES: that
 * would read the floats).  Same argument checks and status codes as the entry point itself; only the
 * layouts are looked at, no pointer is dereferenced.
 *   floats : the float tensor (input of quantize, output of dequantize), typed `dtype`
 *   values : the quantized tensor */
cq_status cq_plan_kind(cq_op op, const cq_tensor* floats, const cq_tensor* values, const cq_tensor* scale,
                       const cq_tensor* out_scale, const cq_scheme* scheme, cq_dtype dtype,
                       uint32_t* family);

/* ---- diagnostics ---- */
const char* cq_strerror(cq_status status);
/* hipError_t of the most recent failed HIP call on the calling thread (0 if none). */
int cq_last_hip_error(void);
uint32_t cq_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* CUBEK_QUANT_H */
