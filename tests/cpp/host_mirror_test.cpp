// Exercises include/axonml_quant.hpp the way the reference crate's own unit tests exercise its API
// (crates/axonml-quant/src/{types,quantize,dequantize}.rs `mod tests`).  Exit code 0 = all checks passed,
// 77 = no usable GPU (Device::open returned nullopt, as CudaBackend::new does), 1 = a check failed.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "axonml_quant.hpp"

using namespace axonml_quant;

static int failures = 0;
#define CHECK(cond)                                                         \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            failures++;                                                     \
        }                                                                   \
    } while (0)

template <class F>
static bool throws(QuantError::Kind kind, F f) {
    try {
        f();
    } catch (const QuantError &e) {
        return e.kind == kind;
    }
    return false;
}

int main() {
    // type registry: types.rs:45-120
    CHECK(block_size(QuantType::Q8_0) == 32 && bytes_per_block(QuantType::Q8_0) == 34);
    CHECK(bytes_per_block(QuantType::Q4_0) == 18 && bytes_per_block(QuantType::Q4_1) == 20);
    CHECK(block_size(QuantType::Q4_K) == 256 && bytes_per_block(QuantType::Q4_K) == 144);
    CHECK(bytes_per_block(QuantType::Q6_K) == 210 && bytes_per_block(QuantType::Q5_K) == 176 && bits_per_value(QuantType::Q6_K) == 6);
    CHECK(quant_type_from_str("q6_k") == QuantType::Q6_K && to_string(QuantType::Q5_K) == "Q5_K");
    CHECK(quant_type_from_str("int8") == QuantType::Q8_0 && quant_type_from_str("Q4_0") == QuantType::Q4_0);
    CHECK(throws(QuantError::Kind::InvalidQuantType, [] { quant_type_from_str("q3_k"); }));
    CHECK(to_string(QuantType::Q4_1) == "Q4_1");

    std::optional<Device> maybe = Device::open(0);
    if (!maybe) {
        std::printf("no usable GPU: %s\n", axq_last_error(nullptr));
        CHECK(throws(QuantError::Kind::Device, [] { Device d(0); }));
        return failures ? 1 : 77;
    }
    Device dev = *maybe;
    std::printf("device: %s\n", dev.name().c_str());

    // quantize.rs:294-313: 8 values -> 1 block, 64 values -> 2 blocks
    std::vector<float> v8(8), v64(64);
    for (int i = 0; i < 8; i++) v8[i] = (float)(i + 1);
    for (int i = 0; i < 64; i++) v64[i] = (float)i / 10.0f;
    CHECK(quantize_tensor(dev, v8, {8}, QuantType::Q8_0).num_blocks() == 1);
    QuantizedTensor q8 = quantize_tensor(dev, v64, {64}, QuantType::Q8_0);
    CHECK(q8.num_blocks() == 2 && q8.size_bytes() == 68);

    // dequantize.rs:204-272: round-trip tolerances
    std::vector<float> back = dequantize_tensor(dev, q8);
    for (int i = 0; i < 64; i++) CHECK(std::fabs(back[i] - v64[i]) < 0.1f);
    QuantizedTensor q4 = quantize_tensor(dev, v64, {64}, QuantType::Q4_0);
    back = dequantize_tensor(dev, q4);
    float worst = 0;
    for (int i = 0; i < 64; i++) worst = std::fmax(worst, std::fabs(back[i] - v64[i]));
    CHECK(worst < 2.0f);
    std::vector<float> h = {1.0f, 2.5f, -3.0f, 4.25f};
    back = dequantize_tensor(dev, quantize_tensor(dev, h, {4}, QuantType::F16));
    for (int i = 0; i < 4; i++) CHECK(std::fabs(back[i] - h[i]) < 0.01f);
    back = dequantize_tensor(dev, quantize_tensor(dev, h, {4}, QuantType::F32));
    CHECK(std::memcmp(back.data(), h.data(), 16) == 0);
    // quantize.rs:324-335: compression ordering
    CHECK(q4.compression_ratio() > q8.compression_ratio());

    // quantize.rs:100,139: an all-zero block gets scale 1.0 (f16 0x3C00); Q4_0 codes are 8 | 8 << 4
    std::vector<float> zeros(32, 0.0f);
    QuantizedTensor z8 = quantize_tensor(dev, zeros, {32}, QuantType::Q8_0);
    CHECK(z8.blocks[0] == 0x00 && z8.blocks[1] == 0x3C && z8.blocks[2] == 0);
    QuantizedTensor z4 = quantize_tensor(dev, zeros, {32}, QuantType::Q4_0);
    CHECK(z4.blocks[1] == 0x3C && z4.blocks[2] == 0x88 && z4.blocks[17] == 0x88);
    CHECK(dequantize_block(dev, z4.blocks.data(), 18, QuantType::Q4_0).size() == 32);

    // quantized matmul against a hand-computable case: W row r = (r + 1) * ones, x = ones -> y_r = 64 (r + 1)
    // (Q8_0 represents these rows exactly: every block is constant, scale = value / 127, code 127)
    const size_t N = 4, K = 64;
    std::vector<float> w(N * K), x(2 * K);
    for (size_t r = 0; r < N; r++)
        for (size_t k = 0; k < K; k++) w[r * K + k] = (float)(r + 1);
    for (size_t k = 0; k < K; k++) { x[k] = 1.0f; x[K + k] = (k % 2) ? -1.0f : 1.0f; }
    QuantizedTensor wq = quantize_tensor(dev, w, {N, K}, QuantType::Q8_0);
    DeviceWeight dw(dev, wq);
    std::vector<float> y = quantized_matmul(x, 2, dw);
    for (size_t r = 0; r < N; r++) {
        CHECK(std::fabs(y[r] - 64.0f * (float)(r + 1)) <= 64.0f * (float)(r + 1) * 1e-3f);
        CHECK(std::fabs(y[N + r]) <= 1e-3f * 64.0f); // alternating signs cancel
    }
    std::vector<float> bias = {0.5f, -1.0f, 2.0f, 0.0f};
    QuantizedLinear lin(dev, wq, bias);
    std::vector<float> yb = lin.forward(x);
    for (size_t r = 0; r < N; r++) CHECK(std::fabs(yb[r] - (y[r] + bias[r])) <= 1e-4f * std::fabs(y[r]) + 1e-5f);

    // error behaviour: error.rs variants
    CHECK(throws(QuantError::Kind::ShapeMismatch, [&] { quantized_matmul(x, 3, dw); }));
    CHECK(throws(QuantError::Kind::DataLengthMismatch, [&] { QuantizedTensor bad({64}, QuantType::Q8_0, std::vector<uint8_t>(67)); }));
    CHECK(throws(QuantError::Kind::ShapeMismatch, [&] { quantize_tensor(dev, v8, {9}, QuantType::Q8_0); }));
    CHECK(std::fabs(compute_quantization_error(v64.data(), v64.data(), 64)) == 0.0f);

    std::printf(failures ? "host mirror: %d check(s) failed\n" : "host mirror: all checks passed\n", failures);
    return failures ? 1 : 0;
}
