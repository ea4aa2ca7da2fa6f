// A consumer of include/cubek_quant_device.hpp: kernels that read PACKED weights and
// dequantize in registers (what the reference's matmul does through the crate's pub
// #[cube] functions, crates/cubek-quant/src/dequantize.rs:20-79).
//   1. dequantize-on-read of a whole tensor must equal cq_dequantize bit for bit;
//   2. a fused GEMV  y = dequant(W) * v  must equal the GEMV over cq_dequantize's output.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/cubek_quant.hpp"
#include "../../include/cubek_quant_device.hpp"

using namespace cubek_quant;
using namespace cubek_quant::scheme;
namespace dev = cubek_quant::device;

#define HIP_OK(x)                                                                       \
    do {                                                                                \
        hipError_t e_ = (x);                                                            \
        if (e_ != hipSuccess) {                                                         \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(2);                                                               \
        }                                                                               \
    } while (0)

template <dev::Float kF, int kBits>
__global__ void dequant_on_read(const uint32_t* words, const float* scales, dev::ScalesLayout layout, uint64_t num_words,
                                float* out) {
    uint64_t p = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= num_words) return;
    float v[32 / kBits];
    dev::dequantize_symmetric_packed_values<kF, kBits>(p, words, scales, layout, v);
    for (int i = 0; i < 32 / kBits; i++) out[p * (32 / kBits) + i] = v[i];
}

// y[r] = sum_c dequant(W[r, c]) * x[c]; one wave per row, packed weights never materialised.
template <dev::Float kF, int kBits>
__global__ void gemv_packed(const uint32_t* words, const float* scales, dev::ScalesLayout layout, uint32_t cols,
                            const float* x, float* y) {
    constexpr int nq = 32 / kBits;
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    const uint32_t words_per_row = cols / nq;
    float acc = 0.0f;
    for (uint32_t w = lane; w < words_per_row; w += 64) {
        float v[nq];
        dev::dequantize_symmetric_packed_values<kF, kBits>(static_cast<uint64_t>(row) * words_per_row + w, words, scales,
                                                          layout, v);
        for (int i = 0; i < nq; i++) acc += v[i] * x[w * nq + i];
    }
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) y[row] = acc;
}

static int failures = 0;
static void report(const char* name, bool ok) {
    std::printf("%s %s\n", ok ? "PASS" : "FAIL", name);
    std::fflush(stdout);
    failures += !ok;
}

template <class T>
static T* to_device(const std::vector<T>& h) {
    T* p;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&p), h.size() * sizeof(T)));
    HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return p;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}
static float bf16_to_f32(uint16_t h) {
    uint32_t u = static_cast<uint32_t>(h) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

template <dev::Float kF, int kBits>
static void run_case(const char* name, QuantValue value, std::vector<uint64_t> shape, std::vector<uint8_t> block) {
    const bool is_bf16 = kF == dev::Float::BF16;
    const ElemType elem = is_bf16 ? ElemType::BF16 : ElemType::F32;
    const size_t esize = is_bf16 ? 2 : 4;
    uint64_t n = 1;
    for (auto s : shape) n *= s;
    const uint64_t cols = shape.back(), rows = n / cols;
    // seeded input
    std::vector<float> hx(n);
    uint32_t seed = 99;
    for (auto& v : hx) {
        seed = seed * 1664525u + 1013904223u;
        v = (static_cast<int>(seed >> 9) % 4001 - 2000) * 1e-4f;
        if (is_bf16) v = bf16_to_f32(f32_to_bf16(v));
    }
    void* d_in;
    if (is_bf16) {
        std::vector<uint16_t> hb(n);
        for (uint64_t i = 0; i < n; i++) hb[i] = f32_to_bf16(hx[i]);
        d_in = to_device(hb);
    } else {
        d_in = to_device(hx);
    }
    QuantScheme scheme = QuantScheme::default_().with_value(value).with_level(QuantLevel::block(block));
    const uint64_t nq = scheme.num_quants();
    std::vector<uint8_t> blk = scheme.level.block_size.to_dim_vec(shape.size());
    std::vector<uint64_t> pshape = shape, sshape = shape;
    pshape.back() /= nq;
    uint64_t ns = 1;
    for (size_t d = 0; d < shape.size(); d++) {
        sshape[d] = shape[d] / blk[d];
        ns *= sshape[d];
    }
    uint32_t* d_words;
    float *d_scales, *d_ref_raw, *d_got, *d_v, *d_y;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_words), n / nq * 4));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_scales), ns * 4));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_ref_raw), n * esize));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_got), n * 4));
    auto t_in = TensorHandleRef::contiguous(d_in, shape, esize);
    auto t_words = TensorHandleRef::contiguous(d_words, pshape, 4);
    auto t_scales = TensorHandleRef::contiguous(d_scales, sshape, 4);
    auto t_ref = TensorHandleRef::contiguous(d_ref_raw, shape, esize);
    ComputeClient client;
    quantize::launch_dynamic(client, t_in, t_words, t_scales, scheme, elem);
    dequantize::launch_ref(client, t_words, t_ref, t_scales, scheme, elem);

    // as the reference's scales_layout(client, values, scales, 1, scheme): from the quantized tensor's shape
    const dev::ScalesLayout layout =
        dev::scales_layout(pshape.data(), static_cast<uint32_t>(pshape.size()), static_cast<uint32_t>(nq),
                           t_scales.strides.data(), block.data(), static_cast<uint32_t>(block.size()));
    const uint64_t num_words = n / nq;
    hipLaunchKernelGGL((dequant_on_read<kF, kBits>), dim3(static_cast<uint32_t>((num_words + 255) / 256)), dim3(256), 0, 0,
                       d_words, d_scales, layout, num_words, d_got);
    HIP_OK(hipDeviceSynchronize());
    std::vector<float> got(n), ref(n);
    HIP_OK(hipMemcpy(got.data(), d_got, n * 4, hipMemcpyDeviceToHost));
    if (is_bf16) {
        std::vector<uint16_t> rb(n);
        HIP_OK(hipMemcpy(rb.data(), d_ref_raw, n * 2, hipMemcpyDeviceToHost));
        for (uint64_t i = 0; i < n; i++) ref[i] = bf16_to_f32(rb[i]);
    } else {
        HIP_OK(hipMemcpy(ref.data(), d_ref_raw, n * 4, hipMemcpyDeviceToHost));
    }
    bool same = std::memcmp(got.data(), ref.data(), n * 4) == 0;
    report((std::string(name) + "::dequantize_on_read_equals_cq_dequantize").c_str(), same);

    // fused GEMV over the packed weights (2-D view rows x cols; the layout still sees the N-D shape)
    std::vector<float> hv(cols);
    for (uint64_t c = 0; c < cols; c++) hv[c] = 0.5f - static_cast<float>(c % 7) * 0.125f;
    d_v = to_device(hv);
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_y), rows * 4));
    hipLaunchKernelGGL((gemv_packed<kF, kBits>), dim3(static_cast<uint32_t>(rows)), dim3(64), 0, 0, d_words, d_scales, layout,
                       static_cast<uint32_t>(cols), d_v, d_y);
    HIP_OK(hipDeviceSynchronize());
    std::vector<float> y(rows);
    HIP_OK(hipMemcpy(y.data(), d_y, rows * 4, hipMemcpyDeviceToHost));
    bool ok = true;
    for (uint64_t r = 0; r < rows && ok; r++) {
        double want = 0, mag = 0;
        for (uint64_t c = 0; c < cols; c++) {
            want += static_cast<double>(ref[r * cols + c]) * hv[c];
            mag += std::fabs(static_cast<double>(ref[r * cols + c]) * hv[c]);
        }
        ok = std::fabs(y[r] - want) <= 1e-5 * mag + 1e-12;  // f32 accumulation order only
    }
    report((std::string(name) + "::fused_gemv_over_packed_weights").c_str(), ok);
    for (void* p : {d_in, (void*)d_words, (void*)d_scales, (void*)d_ref_raw, (void*)d_got, (void*)d_v, (void*)d_y}) (void)hipFree(p);
}

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
        std::printf("no GPU\n");
        return 3;
    }
    run_case<dev::Float::BF16, 4>("bf16_q4s_b32", QuantValue::Q4S, {64, 512}, {32});
    run_case<dev::Float::BF16, 8>("bf16_q8s_b32", QuantValue::Q8S, {64, 512}, {32});
    run_case<dev::Float::F32, 2>("f32_q2s_b64", QuantValue::Q2S, {32, 256}, {64});
    run_case<dev::Float::F32, 4>("f32_q4f_nd_2x3x16", QuantValue::Q4F, {4, 6, 64}, {2, 3, 16});
    run_case<dev::Float::BF16, 4>("bf16_e2m1_b32", QuantValue::E2M1, {16, 1024}, {32});
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}
