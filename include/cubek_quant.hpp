// cubek_quant.hpp — C++ host layer over the C ABI (cubek_quant.h), header only.
//
// It keeps the API surface of the reference crate for this path, name for name:
//   cubek_quant::scheme::{QuantScheme, QuantValue, QuantStore, QuantLevel, QuantParam, QuantMode, BlockSize}
//       (re-exported at crates/cubek-quant/src/lib.rs:14; builder calls as in
//        tests/suite/symmetric.rs:60-66)
//   cubek_quant::quantize::launch_ref     (src/quantize.rs:174-182)
//   cubek_quant::dequantize::launch_ref   (src/dequantize.rs:171-178)
// Error behaviour: where the reference panics (unsupported scheme, block size
// not divisible: src/quantize.rs:203-206,218,273,324; src/lib.rs:28-31) this
// layer throws cubek_quant::Panic; a failed launch (the reference's
// Err(LaunchError)) throws cubek_quant::LaunchError; malformed arguments the
// reference does not check throw std::invalid_argument.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "cubek_quant.h"

namespace cubek_quant {

struct Panic : std::logic_error {
    using std::logic_error::logic_error;
};
struct LaunchError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

namespace scheme {

// E2M1Ocp is an extension without a counterpart in the reference (see CQ_VALUE_E2M1_OCP in cubek_quant.h).
enum class QuantValue : uint8_t { Q8F = 0, Q8S, Q4F, Q4S, Q2F, Q2S, E2M1, E4M3, E5M2, E2M1Ocp };
enum class QuantParam : uint8_t { F32 = 0, F16, BF16 };
enum class QuantStore : uint8_t { U32 = 0, Native };
enum class QuantMode : uint8_t { Symmetric = 0 };

inline size_t size_bits(QuantValue v) { return cq_value_size_bits(static_cast<uint8_t>(v)); }
// (q_min, q_max) as used by the scale rule 2*absmax/(q_max-q_min), tests/suite/symmetric.rs:35-37
inline std::pair<float, float> range(QuantValue v) {
    float lo = 0, hi = 0;
    cq_value_range(static_cast<uint8_t>(v), &lo, &hi);
    return {lo, hi};
}

class BlockSize {
public:
    static constexpr size_t MAX_DIMS = CQ_MAX_BLOCK_DIMS;
    BlockSize() = default;
    BlockSize(std::initializer_list<uint8_t> dims) { assign(dims.begin(), dims.size()); }
    explicit BlockSize(const std::vector<uint8_t>& dims) { assign(dims.data(), dims.size()); }
    const uint8_t* data() const { return storage_.data(); }
    size_t len() const { return len_; }
    std::vector<uint8_t> as_slice() const { return {storage_.begin(), storage_.begin() + len_}; }
    // left-padded with 1s to `rank` entries (src/layout/scales.rs:239)
    std::vector<uint8_t> to_dim_vec(size_t rank) const {
        if (rank < len_) throw std::invalid_argument("block rank exceeds tensor rank");
        std::vector<uint8_t> out(rank - len_, 1);
        out.insert(out.end(), storage_.begin(), storage_.begin() + len_);
        return out;
    }
    size_t num_elements() const {
        size_t n = 1;
        for (size_t i = 0; i < len_; i++) n *= storage_[i];
        return n;
    }

private:
    void assign(const uint8_t* p, size_t n) {
        if (n < 1 || n > MAX_DIMS) throw std::invalid_argument("block size needs 1..5 dimensions");
        for (size_t i = 0; i < n; i++) {
            if (p[i] == 0) throw std::invalid_argument("block extents must be >= 1");
            storage_[i] = p[i];
        }
        len_ = static_cast<uint8_t>(n);
    }
    std::array<uint8_t, MAX_DIMS> storage_{};
    uint8_t len_ = 0;
};

struct QuantLevel {
    bool is_block = false;
    BlockSize block_size;
    static QuantLevel Tensor() { return {}; }
    static QuantLevel block(std::initializer_list<uint8_t> dims) { return {true, BlockSize(dims)}; }
    static QuantLevel block(const std::vector<uint8_t>& dims) { return {true, BlockSize(dims)}; }
};

struct QuantScheme {
    QuantValue value = QuantValue::Q8F;
    QuantParam param = QuantParam::F32;
    QuantStore store = QuantStore::U32;
    QuantLevel level = QuantLevel::Tensor();
    QuantMode mode = QuantMode::Symmetric;

    static QuantScheme default_() { return {}; }
    QuantScheme with_level(QuantLevel l) const { auto s = *this; s.level = l; return s; }
    QuantScheme with_mode(QuantMode m) const { auto s = *this; s.mode = m; return s; }
    QuantScheme with_value(QuantValue v) const { auto s = *this; s.value = v; return s; }
    QuantScheme with_store(QuantStore st) const { auto s = *this; s.store = st; return s; }
    QuantScheme with_param(QuantParam p) const { auto s = *this; s.param = p; return s; }

    size_t size_bits_value() const { return size_bits(value); }
    size_t size_bits_stored() const { return store == QuantStore::U32 ? 32 : size_bits(value); }
    size_t num_quants() const {
        cq_scheme c = to_c();
        return cq_scheme_num_quants(&c);
    }
    cq_scheme to_c() const {
        cq_scheme c{};
        c.value = static_cast<uint8_t>(value);
        c.param = static_cast<uint8_t>(param);
        c.store = static_cast<uint8_t>(store);
        c.level = level.is_block ? CQ_LEVEL_BLOCK : CQ_LEVEL_TENSOR;
        c.mode = static_cast<uint8_t>(mode);
        c.block_rank = level.is_block ? static_cast<uint8_t>(level.block_size.len()) : 0;
        for (size_t i = 0; i < c.block_rank; i++) c.block[i] = level.block_size.data()[i];
        return c;
    }
};

}  // namespace scheme

// Float element types (the reference passes ElemType / StorageType); Flex32 is stored as f32.
enum class ElemType : int { F32 = CQ_F32, F16 = CQ_F16, BF16 = CQ_BF16, Flex32 = CQ_F32 };

// Borrowed device tensor: handle, shape, strides (elements), element size —
// the fields of the reference's TensorHandleRef.
struct TensorHandleRef {
    void* handle = nullptr;
    std::vector<uint64_t> shape;
    std::vector<uint64_t> strides;
    size_t elem_size = 0;

    // contiguous row-major tensor
    static TensorHandleRef contiguous(void* ptr, std::vector<uint64_t> shape, size_t elem_size) {
        TensorHandleRef t;
        t.handle = ptr;
        t.strides.assign(shape.size(), 1);
        for (size_t d = shape.size(); d-- > 1;) t.strides[d - 1] = t.strides[d] * shape[d];
        t.shape = std::move(shape);
        t.elem_size = elem_size;
        return t;
    }
    cq_tensor as_c() const {
        return cq_tensor{handle, shape.data(), strides.data(), static_cast<uint32_t>(shape.size()),
                         static_cast<uint32_t>(elem_size)};
    }
};

// Stands for ComputeClient<R>: the HIP stream launches are ordered on.
struct ComputeClient {
    cq_stream_t stream = nullptr;
};

namespace detail {
inline void check(cq_status st, const scheme::QuantScheme& s) {
    switch (st) {
        case CQ_OK: return;
        case CQ_ERR_UNSUPPORTED_SCHEME:
            throw Panic("Unsupported quantization scheme (value " + std::to_string(int(s.value)) + ", store " +
                        std::to_string(int(s.store)) + ")");
        case CQ_ERR_BLOCK_NOT_DIVISIBLE:
            throw Panic("Block size must be divisible by " + std::to_string(s.num_quants()));
        case CQ_ERR_HIP:
            throw LaunchError(std::string(cq_strerror(st)) + " (hipError_t " + std::to_string(cq_last_hip_error()) + ")");
        default: throw std::invalid_argument(cq_strerror(st));
    }
}
}  // namespace detail

namespace quantize {
// cubek_quant::quantize::launch_ref (src/quantize.rs:174-182)
inline void launch_ref(const ComputeClient& client, const TensorHandleRef& input, const TensorHandleRef& output,
                       const TensorHandleRef& scale, const TensorHandleRef& out_scale,
                       const scheme::QuantScheme& scheme, ElemType input_elem) {
    cq_tensor i = input.as_c(), o = output.as_c(), s = scale.as_c(), os = out_scale.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_quantize(client.stream, &i, &o, &s, &os, &c, static_cast<cq_dtype>(input_elem)), scheme);
}
inline size_t workspace_bytes(const scheme::QuantScheme& scheme, uint64_t num_elements) {
    cq_scheme c = scheme.to_c();
    return cq_workspace_bytes(&c, num_elements);
}
// scale = 2*absmax/(q_max-q_min), typed like the input (tests/suite/symmetric.rs:35-38,156-179)
inline void compute_scales(const ComputeClient& client, const TensorHandleRef& input, const TensorHandleRef& scales,
                           const scheme::QuantScheme& scheme, ElemType input_elem, void* workspace = nullptr,
                           size_t workspace_size = 0) {
    cq_tensor i = input.as_c(), s = scales.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_compute_scales(client.stream, &i, &s, &c, static_cast<cq_dtype>(input_elem), workspace,
                                    workspace_size), scheme);
}
// fused abs-max + scale + quantize
inline void launch_dynamic(const ComputeClient& client, const TensorHandleRef& input, const TensorHandleRef& output,
                           const TensorHandleRef& out_scale, const scheme::QuantScheme& scheme, ElemType input_elem,
                           void* workspace = nullptr, size_t workspace_size = 0) {
    cq_tensor i = input.as_c(), o = output.as_c(), os = out_scale.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_quantize_dynamic(client.stream, &i, &o, &os, &c, static_cast<cq_dtype>(input_elem), workspace,
                                      workspace_size), scheme);
}
// the same without a workspace: the scratch memory is an array inside the library (one per GPU,
// shared by all calls on that GPU), for callers that cannot allocate device memory
inline void launch_dynamic_static(const ComputeClient& client, const TensorHandleRef& input, const TensorHandleRef& output,
                                  const TensorHandleRef& out_scale, const scheme::QuantScheme& scheme, ElemType input_elem) {
    cq_tensor i = input.as_c(), o = output.as_c(), os = out_scale.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_quantize_dynamic_static(client.stream, &i, &o, &os, &c, static_cast<cq_dtype>(input_elem)), scheme);
}
}  // namespace quantize

namespace dequantize {
// cubek_quant::dequantize::launch_ref (src/dequantize.rs:171-178); `input_dtype`
// is the float type of `output`, as in the reference.
inline void launch_ref(const ComputeClient& client, const TensorHandleRef& values, const TensorHandleRef& output,
                       const TensorHandleRef& params, const scheme::QuantScheme& scheme, ElemType input_dtype) {
    cq_tensor v = values.as_c(), o = output.as_c(), p = params.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_dequantize(client.stream, &v, &o, &p, &c, static_cast<cq_dtype>(input_dtype)), scheme);
}
}  // namespace dequantize

namespace reduce {
// cubek_reduce::ReduceError (crates/cubek-reduce/src/error.rs:6-36), the variants this path can raise.
struct ReduceError : std::runtime_error {
    enum Kind { InvalidAxis, MismatchShape, Launch } kind;
    ReduceError(Kind k, const std::string& what) : std::runtime_error(what), kind(k) {}
};

inline size_t workspace_bytes(const TensorHandleRef& input, size_t axis, ElemType dtype) {
    cq_tensor i = input.as_c();
    return cq_reduce_workspace_bytes(&i, static_cast<uint32_t>(axis), static_cast<cq_dtype>(dtype));
}

// cubek_reduce::reduce::<R, MaxAbs> (crates/cubek-reduce/src/lib.rs:93-131): `output` has the
// shape of `input` with extent 1 on `axis`.  The reference returns Err(ReduceError); here it is thrown.
inline void max_abs(const ComputeClient& client, const TensorHandleRef& input, const TensorHandleRef& output,
                    size_t axis, ElemType dtype, void* workspace = nullptr, size_t workspace_size = 0) {
    cq_tensor i = input.as_c(), o = output.as_c();
    const cq_status st = cq_reduce_max_abs(client.stream, &i, &o, static_cast<uint32_t>(axis),
                                           static_cast<cq_dtype>(dtype), workspace, workspace_size);
    switch (st) {
        case CQ_OK: return;
        case CQ_ERR_INVALID_AXIS:
            throw ReduceError(ReduceError::InvalidAxis, "The provided axis (" + std::to_string(axis) +
                                                            ") must be smaller than the input tensor rank (" +
                                                            std::to_string(input.shape.size()) + ").");
        case CQ_ERR_SHAPE_MISMATCH:
            throw ReduceError(ReduceError::MismatchShape, "The output shape is not the input shape with 1 on the axis.");
        case CQ_ERR_HIP:
            throw ReduceError(ReduceError::Launch, std::string(cq_strerror(st)) + " (hipError_t " +
                                                       std::to_string(cq_last_hip_error()) + ")");
        default: throw std::invalid_argument(cq_strerror(st));
    }
}
}  // namespace reduce

namespace contiguous {
// cubecl_std::tensor::into_contiguous_packed_ref as cubek-matmul uses it on quantized operands
// (crates/cubek-matmul/src/base.rs:505-529): `shape` is the logical shape, `packing` the values per
// stored element; `output` is contiguous with the last dimension of `shape` divided by `packing`.
inline void into_contiguous_packed_ref(const ComputeClient& client, const TensorHandleRef& input,
                                       const TensorHandleRef& output, const std::vector<uint64_t>& shape,
                                       uint32_t packing) {
    cq_tensor i = input.as_c(), o = output.as_c();
    const cq_status st = cq_into_contiguous_packed(client.stream, &i, &o, shape.data(),
                                                   static_cast<uint32_t>(shape.size()), packing);
    if (st == CQ_OK) return;
    if (st == CQ_ERR_HIP)
        throw LaunchError(std::string(cq_strerror(st)) + " (hipError_t " + std::to_string(cq_last_hip_error()) + ")");
    throw std::invalid_argument(cq_strerror(st));
}
}  // namespace contiguous

namespace matvec {
// The matrix-vector case of a matmul with a quantized operand (MatmulInputHandle::Quantized,
// crates/cubek-matmul/src/base.rs:309-317): y = dequantize(values, params) * x with the weights read once in
// their stored form.  `values` [rows, cols / num_quants] (U32 store) or the byte tensor of the native store,
// `x` [cols] or [vectors, cols] of `elem`, `y` [rows] or [vectors, rows] of `y_elem`.
inline void launch_ref(const ComputeClient& client, const TensorHandleRef& values, const TensorHandleRef& params,
                       const scheme::QuantScheme& scheme, const TensorHandleRef& x, const TensorHandleRef& y, ElemType elem,
                       ElemType y_elem) {
    cq_tensor v = values.as_c(), p = params.as_c(), xs = x.as_c(), ys = y.as_c();
    cq_scheme c = scheme.to_c();
    detail::check(cq_gemv_quantized(client.stream, &v, &p, &c, &xs, &ys, static_cast<cq_dtype>(elem),
                                    static_cast<cq_dtype>(y_elem)),
                  scheme);
}
}  // namespace matvec

}  // namespace cubek_quant
