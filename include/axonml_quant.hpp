// axonml_quant.hpp -- C++ host mirror of the `axonml-quant` crate's public API over the axq C ABI.
//
// The reference host side is Rust (crates/axonml-quant/src/lib.rs:35-49 re-exports the names below).  This
// header keeps those names, argument meanings and error behaviour for C++ callers; every operation runs on
// the device through libaxq.so (include/axq.h).  There is no CPU path: constructing a Device on a machine
// without a gfx950 GPU throws.
//
//   reference                                   here
//   QuantType (types.rs:17-120)                 axonml_quant::QuantType + free functions of the same names
//   QuantError / QuantResult (error.rs:11-57)   axonml_quant::QuantError (exception carrying the variant)
//   QuantizedTensor (types.rs:296-334)          axonml_quant::QuantizedTensor (flat `to_bytes` image)
//   quantize_tensor / quantize_model            same names (quantize.rs:36-75)
//   dequantize_tensor / dequantize_block        same names (dequantize.rs:34-65)
//   compute_quantization_error (quantize.rs:235-248)   same name
//   x.matmul(dequantize_tensor(w).t()) + bias   quantized_matmul / QuantizedLinear::forward (nn/src/layers/linear.rs:104-140)
//   CudaBackend::new -> Option (cuda.rs:69-81)  Device::open -> std::optional<Device>
#pragma once
#include <cmath>
#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "axq.h"

namespace axonml_quant {

constexpr size_t DEFAULT_BLOCK_SIZE = 32; // lib.rs:46
constexpr size_t MAX_BLOCK_SIZE = 256;    // lib.rs:49

// ---- QuantType (types.rs:17-41), discriminants equal to axq_type -----------------------------------
enum class QuantType : int { Q8_0 = AXQ_Q8_0, Q4_0 = AXQ_Q4_0, Q4_1 = AXQ_Q4_1, Q5_0 = AXQ_Q5_0, Q5_1 = AXQ_Q5_1,
                             F16 = AXQ_F16, F32 = AXQ_F32, Q4_K = AXQ_Q4_K, Q6_K = AXQ_Q6_K, Q5_K = AXQ_Q5_K };
inline size_t block_size(QuantType t) { return axq_type_block_size((int)t); }           // types.rs:45-54
inline size_t bytes_per_block(QuantType t) { return axq_type_bytes_per_block((int)t); } // :57-67
inline size_t bits_per_value(QuantType t) { return axq_type_bits_per_value((int)t); }   // :70-78
inline bool is_block_quantized(QuantType t) { return axq_type_is_block_quantized((int)t) != 0; } // :86-91
inline std::string to_string(QuantType t) { return axq_type_name((int)t); }             // Display, :108-120
inline double compression_ratio(QuantType t) { return 32.0 / (double)bits_per_value(t); } // :81-83

// ---- QuantError (error.rs:14-57) --------------------------------------------------------------------
class QuantError : public std::runtime_error {
  public:
    enum class Kind { InvalidBlockSize, InvalidQuantType, ShapeMismatch, DataLengthMismatch, CalibrationError, Overflow,
                      InvalidData, TensorConversion, Device };
    QuantError(Kind k, const std::string &msg) : std::runtime_error(msg), kind(k) {}
    Kind kind;
};

inline QuantType quant_type_from_str(const std::string &s) { // QuantType::from_str (types.rs:94-105)
    int t = axq_type_from_str(s.c_str());
    if (t < 0) throw QuantError(QuantError::Kind::InvalidQuantType, "Invalid quantization type: " + s);
    return (QuantType)t;
}

namespace detail {
inline QuantError::Kind kind_of(int status) {
    switch (status) {
    case AXQ_ERR_INVALID_BLOCK_SIZE: return QuantError::Kind::InvalidBlockSize;
    case AXQ_ERR_INVALID_QUANT_TYPE: return QuantError::Kind::InvalidQuantType;
    case AXQ_ERR_SHAPE_MISMATCH: return QuantError::Kind::ShapeMismatch;
    case AXQ_ERR_DATA_LENGTH_MISMATCH: return QuantError::Kind::DataLengthMismatch;
    case AXQ_ERR_CALIBRATION: return QuantError::Kind::CalibrationError;
    case AXQ_ERR_OVERFLOW: return QuantError::Kind::Overflow;
    case AXQ_ERR_INVALID_DATA: return QuantError::Kind::InvalidData;
    case AXQ_ERR_TENSOR_CONVERSION: return QuantError::Kind::TensorConversion;
    default: return QuantError::Kind::Device; // the CudaError mirror, -20..-30
    }
}
inline size_t numel_of(const std::vector<size_t> &shape) {
    size_t n = 1;
    for (size_t s : shape) n *= s;
    return n;
}
} // namespace detail

// ---- the device: Backend trait (backends/mod.rs:73-100) narrowed to what this path needs -------------
class Device {
  public:
    static std::optional<Device> open(int index = 0) { // None when there is no usable GPU
        axq_ctx *c = nullptr;
        if (axq_init(index, &c) != AXQ_OK) return std::nullopt;
        return Device(c);
    }
    explicit Device(int index = 0) {
        axq_ctx *c = nullptr;
        int rc = axq_init(index, &c);
        if (rc != AXQ_OK) throw QuantError(QuantError::Kind::Device, axq_last_error(nullptr));
        ctx_.reset(c, axq_destroy);
    }
    axq_ctx *ctx() const { return ctx_.get(); }
    void check(int rc) const {
        if (rc != AXQ_OK) throw QuantError(detail::kind_of(rc), axq_last_error(ctx_.get()));
    }
    std::string name() const {
        axq_device_info_t info;
        check(axq_device_info(ctx_.get(), &info));
        return std::string(info.name) + " (" + info.arch + ")";
    }
    void synchronize() const { check(axq_synchronize(ctx_.get())); }

  private:
    explicit Device(axq_ctx *c) : ctx_(c, axq_destroy) {}
    std::shared_ptr<axq_ctx> ctx_;
};

// ---- QuantizedTensor (types.rs:296-334) --------------------------------------------------------------
struct QuantizedTensor {
    std::vector<size_t> shape;
    QuantType quant_type;
    std::vector<uint8_t> blocks; // the concatenated `to_bytes` images, in block order
    size_t numel;

    QuantizedTensor(std::vector<size_t> shape_, QuantType t, std::vector<uint8_t> data)
        : shape(std::move(shape_)), quant_type(t), blocks(std::move(data)), numel(detail::numel_of(shape)) {
        size_t expect = axq_packed_bytes((int)t, numel);
        if (blocks.size() != expect)
            throw QuantError(QuantError::Kind::DataLengthMismatch,
                             "Data length mismatch: expected " + std::to_string(expect) + ", got " + std::to_string(blocks.size()));
    }
    size_t num_blocks() const { return is_block_quantized(quant_type) ? axq_num_blocks((int)quant_type, numel) : 1; }
    size_t size_bytes() const { return num_blocks() * bytes_per_block(quant_type); } // types.rs:320-322
    double compression_ratio() const { return (double)(numel * 4) / (double)size_bytes(); }
};

// ---- quantize / dequantize ---------------------------------------------------------------------------
inline QuantizedTensor quantize_tensor(const Device &dev, const float *data, const std::vector<size_t> &shape, QuantType t) {
    size_t n = detail::numel_of(shape);
    std::vector<uint8_t> out(axq_packed_bytes((int)t, n));
    dev.check(axq_quantize(dev.ctx(), (int)t, data, n, out.data(), AXQ_MEM_HOST));
    return QuantizedTensor(shape, t, std::move(out));
}
inline QuantizedTensor quantize_tensor(const Device &dev, const std::vector<float> &data, const std::vector<size_t> &shape, QuantType t) {
    if (data.size() != detail::numel_of(shape))
        throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: data length does not match the shape");
    return quantize_tensor(dev, data.data(), shape, t);
}

struct NamedTensor {
    std::string name;
    const float *data;
    std::vector<size_t> shape;
};
// quantize_model (quantize.rs:64-75): the first error aborts.
inline std::vector<std::pair<std::string, QuantizedTensor>> quantize_model(const Device &dev, const std::vector<NamedTensor> &tensors,
                                                                           QuantType t) {
    std::vector<std::pair<std::string, QuantizedTensor>> out;
    out.reserve(tensors.size());
    for (const NamedTensor &nt : tensors) out.emplace_back(nt.name, quantize_tensor(dev, nt.data, nt.shape, t));
    return out;
}

// dequantize_tensor (dequantize.rs:34-54): numel floats, the padded tail of the last block dropped.
inline std::vector<float> dequantize_tensor(const Device &dev, const QuantizedTensor &q) {
    std::vector<float> out(q.numel);
    dev.check(axq_dequantize(dev.ctx(), (int)q.quant_type, q.blocks.data(), q.numel, out.data(), AXQ_MEM_HOST));
    return out;
}
// dequantize_block (dequantize.rs:57-65): one block's byte image -> block_size floats.
inline std::vector<float> dequantize_block(const Device &dev, const uint8_t *block, size_t bytes, QuantType t) {
    size_t n = is_block_quantized(t) ? block_size(t) : bytes / bytes_per_block(t);
    if (is_block_quantized(t) && bytes != bytes_per_block(t))
        throw QuantError(QuantError::Kind::InvalidData, "Invalid quantized data: wrong block length");
    std::vector<float> out(n);
    dev.check(axq_dequantize(dev.ctx(), (int)t, block, n, out.data(), AXQ_MEM_HOST));
    return out;
}
// compute_quantization_error (quantize.rs:235-248): RMSE between a tensor and its round trip.
inline float compute_quantization_error(const float *original, const float *dequantized, size_t n) {
    if (n == 0) return 0.0f;
    float s = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float d = original[i] - dequantized[i];
        s += d * d;
    }
    return std::sqrt(s / (float)n);
}

// ---- device-resident weight and the quantized matmul -------------------------------------------------
class DeviceWeight {
  public:
    DeviceWeight(const Device &dev, const QuantizedTensor &q) : dev_(dev) {
        if (q.shape.size() != 2) throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: a Linear weight is [out, in]");
        axq_weight *w = nullptr;
        dev.check(axq_weight_upload(dev.ctx(), (int)q.quant_type, (int64_t)q.shape[0], (int64_t)q.shape[1], q.blocks.data(),
                                    q.blocks.size(), AXQ_MEM_HOST, &w));
        w_ = w;
        rows_ = q.shape[0];
        k_ = q.shape[1];
    }
    DeviceWeight(const DeviceWeight &) = delete;
    DeviceWeight &operator=(const DeviceWeight &) = delete;
    ~DeviceWeight() { axq_weight_free(dev_.ctx(), w_); }
    const axq_weight *handle() const { return w_; }
    size_t out_features() const { return rows_; }
    size_t in_features() const { return k_; }
    const Device &device() const { return dev_; }

  private:
    Device dev_;
    axq_weight *w_ = nullptr;
    size_t rows_ = 0, k_ = 0;
};

// y[rows, out] = x[rows, in] * W^T (+ bias[out]), f32: what the reference spells
// x.matmul(&dequantize_tensor(&w)?.t()?) followed by the broadcast add of Linear::forward.
inline std::vector<float> quantized_matmul(const std::vector<float> &x, size_t rows, const DeviceWeight &w,
                                           const std::vector<float> *bias = nullptr) {
    if (x.size() != rows * w.in_features())
        throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: x is not [rows, in_features]");
    if (bias && bias->size() != w.out_features())
        throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: bias is not [out_features]");
    std::vector<float> y(rows * w.out_features());
    w.device().check(axq_gemv_f32(w.device().ctx(), w.handle(), x.data(), (int)rows, bias ? bias->data() : nullptr, y.data(),
                                  AXQ_MEM_HOST));
    return y;
}

// Linear::from_weights (nn/src/layers/linear.rs:80-90) with a quantized weight.
class QuantizedLinear {
  public:
    QuantizedLinear(const Device &dev, const QuantizedTensor &weight, std::optional<std::vector<float>> bias = std::nullopt)
        : weight_(dev, weight), bias_(std::move(bias)) {
        if (bias_ && bias_->size() != weight_.out_features())
            throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: bias is not [out_features]");
    }
    // x: [..., in_features] flattened to rows; returns [rows, out_features]
    std::vector<float> forward(const std::vector<float> &x) const {
        if (x.size() % weight_.in_features() != 0)
            throw QuantError(QuantError::Kind::ShapeMismatch, "Shape mismatch: last dimension is not in_features");
        return quantized_matmul(x, x.size() / weight_.in_features(), weight_, bias_ ? &*bias_ : nullptr);
    }
    size_t in_features() const { return weight_.in_features(); }
    size_t out_features() const { return weight_.out_features(); }

  private:
    DeviceWeight weight_;
    std::optional<std::vector<float>> bias_;
};

} // namespace axonml_quant
