// The reference crate's own test suite, case for case, through the C++ host
// layer (include/cubek_quant.hpp): crates/cubek-quant/tests/suite/symmetric.rs
// stamped over {32x32, 16x64} x {Q8F,Q8S,Q4F,Q4S,Q2F,Q2S} (tests/suite/mod.rs:18-52),
// plus the host-layer error behaviour.  Needs a GPU; run by tests/test_gpu_cpp_suite.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/cubek_quant.hpp"

using namespace cubek_quant;
using namespace cubek_quant::scheme;

#define HIP_OK(x)                                                                         \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);   \
            std::exit(2);                                                                 \
        }                                                                                 \
    } while (0)

template <class T>
struct DeviceBuffer {
    T* ptr = nullptr;
    size_t n = 0;
    explicit DeviceBuffer(size_t count) : n(count) {
        HIP_OK(hipMalloc(reinterpret_cast<void**>(&ptr), count * sizeof(T)));
        HIP_OK(hipMemset(ptr, 0, count * sizeof(T)));
    }
    explicit DeviceBuffer(const std::vector<T>& host) : DeviceBuffer(host.size()) {
        HIP_OK(hipMemcpy(ptr, host.data(), n * sizeof(T), hipMemcpyHostToDevice));
    }
    ~DeviceBuffer() { (void)hipFree(ptr); }
    std::vector<T> read() const {
        std::vector<T> h(n);
        HIP_OK(hipMemcpy(h.data(), ptr, n * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

static int failures = 0;
static void report(const std::string& name, bool ok, const std::string& why = "") {
    std::printf("%s %s %s\n", ok ? "PASS" : "FAIL", name.c_str(), why.c_str());
    std::fflush(stdout);
    if (!ok) failures++;
}

// test_quantization_tensor_symmetric (symmetric.rs:24-141)
static void test_quantization_tensor_symmetric(size_t m, size_t n, QuantValue value, const std::string& name) {
    ComputeClient client;
    const size_t num_elems = m * n;
    const float half = static_cast<float>(num_elems) / 2.0f;
    std::vector<float> data(num_elems);
    for (size_t v = 0; v < num_elems; v++) data[v] = static_cast<float>(v) - half;

    auto [q_min, q_max] = range(value);
    const float scale_f32 = (2.0f * half) / (q_max - q_min);

    QuantScheme scheme = QuantScheme::default_()
                             .with_level(QuantLevel::Tensor())
                             .with_mode(QuantMode::Symmetric)
                             .with_value(value)
                             .with_store(QuantStore::U32)
                             .with_param(QuantParam::F32);

    DeviceBuffer<float> input(data), scale(std::vector<float>{scale_f32}), output_f(num_elems), output_scale(1);
    // The shape is from the POV of packed u32s.
    DeviceBuffer<uint32_t> output(num_elems / scheme.num_quants());
    auto t_in = TensorHandleRef::contiguous(input.ptr, {m, n}, 4);
    auto t_out = TensorHandleRef::contiguous(output.ptr, {m, n / scheme.num_quants()}, 4);
    auto t_scale = TensorHandleRef::contiguous(scale.ptr, {1}, 4);
    auto t_out_scale = TensorHandleRef::contiguous(output_scale.ptr, {1}, 4);
    auto t_out_f = TensorHandleRef::contiguous(output_f.ptr, {m, n}, 4);

    quantize::launch_ref(client, t_in, t_out, t_scale, t_out_scale, scheme, ElemType::Flex32);
    dequantize::launch_ref(client, t_out, t_out_f, t_out_scale, scheme, ElemType::F32);
    HIP_OK(hipDeviceSynchronize());
    std::vector<float> restored = output_f.read();

    // Max quantization error = step size / 2
    const float rel_tol = 1e-4f;
    const float max_error = (scale_f32 / 2.0f) * (1.0f + rel_tol);
    bool ok = restored.size() == data.size();
    for (size_t i = 0; ok && i < data.size(); i++) ok = std::fabs(restored[i] - data[i]) <= max_error;
    report(name + "::test_quantization_symmetric_tensor", ok);
}

// test_quantization_block_symmetric (symmetric.rs:143-284)
static void test_quantization_block_symmetric(size_t m, size_t n, QuantValue value, size_t block_size,
                                              const std::string& name) {
    ComputeClient client;
    const size_t num_elems = m * n;
    const float half = static_cast<float>(num_elems) / 2.0f;
    std::vector<float> data(num_elems);
    for (size_t v = 0; v < num_elems; v++) data[v] = (static_cast<float>(v) - half) / static_cast<float>(num_elems);

    auto [q_min, q_max] = range(value);
    const size_t scale_count = num_elems / block_size;
    std::vector<float> scales(scale_count);
    for (size_t block = 0; block < scale_count; block++) {
        float c_max = -INFINITY, c_min = INFINITY;
        for (size_t i = 0; i < block_size; i++) {
            float current = data[block * block_size + i];
            c_max = std::fmax(c_max, current);
            c_min = std::fmin(c_min, current);
        }
        // The bias is assumed to be zero.
        const float rng = 2.0f * std::fmax(std::fabs(c_min), std::fabs(c_max));
        scales[block] = rng / (q_max - q_min);
    }

    QuantScheme scheme = QuantScheme::default_()
                             .with_level(QuantLevel::block({static_cast<uint8_t>(block_size)}))
                             .with_mode(QuantMode::Symmetric)
                             .with_value(value)
                             .with_store(QuantStore::U32)
                             .with_param(QuantParam::F32);

    DeviceBuffer<float> input(data), scale(scales), output_f(num_elems), output_scale(scale_count);
    DeviceBuffer<uint32_t> output(num_elems / scheme.num_quants());
    auto t_in = TensorHandleRef::contiguous(input.ptr, {m, n}, 4);
    auto t_out = TensorHandleRef::contiguous(output.ptr, {m, n / scheme.num_quants()}, 4);
    auto t_scale = TensorHandleRef::contiguous(scale.ptr, {m, n / block_size}, 4);
    auto t_out_scale = TensorHandleRef::contiguous(output_scale.ptr, {m, n / block_size}, 4);
    auto t_out_f = TensorHandleRef::contiguous(output_f.ptr, {m, n}, 4);

    quantize::launch_ref(client, t_in, t_out, t_scale, t_out_scale, scheme, ElemType::Flex32);
    dequantize::launch_ref(client, t_out, t_out_f, t_out_scale, scheme, ElemType::F32);
    HIP_OK(hipDeviceSynchronize());
    std::vector<float> restored = output_f.read();

    bool ok = restored.size() == data.size();
    const float rel_tol = 1e-4f;
    for (size_t i = 0; ok && i < data.size(); i++) {
        const float max_error = (scales[i / block_size] / 2.0f) * (1.0f + rel_tol);
        ok = std::fabs(restored[i] - data[i]) <= max_error;
    }
    // out_scale is the scale tensor cast to the param type (src/quantize.rs:83-98)
    ok = ok && output_scale.read() == scales;

    // the fused path must agree with scales from the host rule
    DeviceBuffer<uint32_t> output_dyn(num_elems / scheme.num_quants());
    DeviceBuffer<float> scale_dyn(scale_count);
    auto t_out_dyn = TensorHandleRef::contiguous(output_dyn.ptr, {m, n / scheme.num_quants()}, 4);
    auto t_scale_dyn = TensorHandleRef::contiguous(scale_dyn.ptr, {m, n / block_size}, 4);
    quantize::launch_dynamic(client, t_in, t_out_dyn, t_scale_dyn, scheme, ElemType::F32);
    HIP_OK(hipDeviceSynchronize());
    ok = ok && output_dyn.read() == output.read() && scale_dyn.read() == scales;
    report(name + "::test_quantization_symmetric_block", ok);
}

static void test_error_behaviour() {
    ComputeClient client;
    DeviceBuffer<float> x(8 * 64), s(8 * 32), os(8 * 32);
    DeviceBuffer<uint32_t> out(8 * 16);
    auto t_x = TensorHandleRef::contiguous(x.ptr, {8, 64}, 4);
    auto t_out = TensorHandleRef::contiguous(out.ptr, {8, 16}, 4);
    // block of 2 with 4 values per u32: the reference asserts (src/lib.rs:28-31)
    {
        auto scheme = QuantScheme::default_().with_value(QuantValue::Q8S).with_level(QuantLevel::block({2}));
        auto t_s = TensorHandleRef::contiguous(s.ptr, {8, 32}, 4);
        auto t_os = TensorHandleRef::contiguous(os.ptr, {8, 32}, 4);
        bool threw = false;
        try {
            quantize::launch_ref(client, t_x, t_out, t_s, t_os, scheme, ElemType::F32);
        } catch (const Panic& e) {
            threw = std::string(e.what()).find("divisible") != std::string::npos;
        }
        report("errors::block_size_not_divisible_panics", threw);
    }
    // Q4S has no native store: the reference panics (src/quantize.rs:213-219)
    {
        auto scheme = QuantScheme::default_().with_value(QuantValue::Q4S).with_store(QuantStore::Native);
        auto t_s = TensorHandleRef::contiguous(s.ptr, {1}, 4);
        bool threw = false;
        try {
            quantize::launch_ref(client, t_x, t_out, t_s, t_s, scheme, ElemType::F32);
        } catch (const Panic&) {
            threw = true;
        }
        report("errors::unsupported_native_value_panics", threw);
    }
    // shapes that do not agree are refused instead of read out of bounds
    {
        auto scheme = QuantScheme::default_().with_value(QuantValue::Q8S);
        auto t_bad = TensorHandleRef::contiguous(out.ptr, {8, 15}, 4);
        auto t_s = TensorHandleRef::contiguous(s.ptr, {1}, 4);
        bool threw = false;
        try {
            quantize::launch_ref(client, t_x, t_bad, t_s, t_s, scheme, ElemType::F32);
        } catch (const std::invalid_argument&) {
            threw = true;
        }
        report("errors::shape_mismatch_is_invalid_argument", threw);
    }
    // scheme helpers
    {
        bool ok = QuantScheme::default_().num_quants() == 4 &&
                  QuantScheme::default_().with_value(QuantValue::Q2S).num_quants() == 16 &&
                  range(QuantValue::Q4F) == std::pair<float, float>(-8.f, 7.f) &&
                  BlockSize({2, 16}).to_dim_vec(4) == std::vector<uint8_t>({1, 1, 2, 16});
        report("scheme::helpers", ok);
    }
}

// MaxAbs along an axis feeding the test's scale rule: per-row abs-max of an [m, n] ramp,
// and the error variants of cubek_reduce::reduce (crates/cubek-reduce/src/lib.rs:101-102).
static void test_reduce_max_abs() {
    ComputeClient client;
    const size_t m = 16, n = 64;
    std::vector<float> data(m * n);
    for (size_t i = 0; i < m * n; i++) data[i] = (i % 2 ? -1.0f : 1.0f) * static_cast<float>(i) / 8.0f;
    DeviceBuffer<float> x(data), rows(m), cols(n);
    auto t_x = TensorHandleRef::contiguous(x.ptr, {m, n}, 4);
    auto t_rows = TensorHandleRef::contiguous(rows.ptr, {m, 1}, 4);
    auto t_cols = TensorHandleRef::contiguous(cols.ptr, {1, n}, 4);
    reduce::max_abs(client, t_x, t_rows, 1, ElemType::F32);
    reduce::max_abs(client, t_x, t_cols, 0, ElemType::F32);
    HIP_OK(hipDeviceSynchronize());
    bool ok = true;
    auto got_rows = rows.read(), got_cols = cols.read();
    for (size_t r = 0; r < m; r++) ok = ok && got_rows[r] == static_cast<float>(r * n + n - 1) / 8.0f;
    for (size_t c = 0; c < n; c++) ok = ok && got_cols[c] == static_cast<float>((m - 1) * n + c) / 8.0f;
    report("reduce::max_abs_rows_and_columns", ok);
    bool bad_axis = false, bad_shape = false;
    try {
        reduce::max_abs(client, t_x, t_rows, 2, ElemType::F32);
    } catch (const reduce::ReduceError& e) {
        bad_axis = e.kind == reduce::ReduceError::InvalidAxis;
    }
    try {
        reduce::max_abs(client, t_x, t_cols, 1, ElemType::F32);
    } catch (const reduce::ReduceError& e) {
        bad_shape = e.kind == reduce::ReduceError::MismatchShape;
    }
    report("reduce::invalid_axis_and_mismatch_shape", bad_axis && bad_shape);
}

// matvec::launch_ref against the dequantized weights times x on the host (f32 throughout)
static void test_matvec() {
    ComputeClient client;
    const size_t m = 16, n = 64, block_size = 32;
    std::vector<float> data(m * n), xs(n);
    for (size_t i = 0; i < m * n; i++) data[i] = std::sin(static_cast<float>(i) * 0.37f);
    for (size_t i = 0; i < n; i++) xs[i] = std::cos(static_cast<float>(i) * 0.11f);
    QuantScheme scheme = QuantScheme::default_()
                             .with_level(QuantLevel::block({static_cast<uint8_t>(block_size)}))
                             .with_value(QuantValue::Q8S)
                             .with_store(QuantStore::U32)
                             .with_param(QuantParam::F32);
    DeviceBuffer<float> input(data), x(xs), scale(m * n / block_size), restored(m * n), y(m);
    DeviceBuffer<uint32_t> words(m * n / scheme.num_quants());
    auto t_in = TensorHandleRef::contiguous(input.ptr, {m, n}, 4);
    auto t_words = TensorHandleRef::contiguous(words.ptr, {m, n / scheme.num_quants()}, 4);
    auto t_scale = TensorHandleRef::contiguous(scale.ptr, {m, n / block_size}, 4);
    auto t_restored = TensorHandleRef::contiguous(restored.ptr, {m, n}, 4);
    auto t_x = TensorHandleRef::contiguous(x.ptr, {n}, 4);
    auto t_y = TensorHandleRef::contiguous(y.ptr, {m}, 4);
    quantize::launch_dynamic(client, t_in, t_words, t_scale, scheme, ElemType::F32);
    dequantize::launch_ref(client, t_words, t_restored, t_scale, scheme, ElemType::F32);
    matvec::launch_ref(client, t_words, t_scale, scheme, t_x, t_y, ElemType::F32, ElemType::F32);
    HIP_OK(hipDeviceSynchronize());
    const std::vector<float> w = restored.read(), got = y.read();
    bool ok = true;
    for (size_t r = 0; r < m; r++) {
        double want = 0.0, mag = 0.0;
        for (size_t c = 0; c < n; c++) {
            want += static_cast<double>(w[r * n + c]) * xs[c];
            mag += std::fabs(static_cast<double>(w[r * n + c]) * xs[c]);
        }
        ok = ok && std::fabs(got[r] - want) <= 2e-5 * mag;
    }
    report("matvec::launch_ref", ok);
}

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
        std::printf("no GPU\n");
        return 3;
    }
    const struct { size_t x, y; const char* name; } sizes[] = {{32, 32, "size32x32"}, {16, 64, "size16x64"}};
    const struct { QuantValue v; const char* name; } values[] = {
        {QuantValue::Q8F, "q8f"}, {QuantValue::Q8S, "q8s"}, {QuantValue::Q4F, "q4f"},
        {QuantValue::Q4S, "q4s"}, {QuantValue::Q2F, "q2f"}, {QuantValue::Q2S, "q2s"}};
    for (const auto& sz : sizes)
        for (const auto& v : values) {
            std::string name = std::string("quant::") + sz.name + "::" + v.name;
            test_quantization_tensor_symmetric(sz.x, sz.y, v.v, name);
            test_quantization_block_symmetric(sz.x, sz.y, v.v, sz.x /* Shape x as block_size */, name);
        }
    test_error_behaviour();
    test_reduce_max_abs();
    test_matvec();
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}
