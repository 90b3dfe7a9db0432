"""Host-side mirror of the ``axonml-quant`` API over the axq C ABI.

Names, argument meaning and error behaviour follow the reference crate
(crates/axonml-quant/src/lib.rs:35-49):

    QuantType, QuantizedTensor, QuantError            types.rs, error.rs
    quantize_tensor, quantize_model                   quantize.rs:36-75
    dequantize_tensor, dequantize_block               dequantize.rs:34-65
    quantized_matmul, QuantizedLinear                 the fused form of
        dequantize_tensor -> Linear::forward (nn/src/layers/linear.rs:104-140)

Every function computes on the GPU through ``libaxq.so``; tensors are numpy
arrays on the host side of the boundary.  Differences from the reference, all
additions: ``QuantType.Q4_K``, ``QuantType.Q5_K`` and ``QuantType.Q6_K`` (GGUF superblocks); Q5_0/Q5_1 have real codecs (the reference aliases
them to Q4_0, quantize.rs:47-50); a ``QuantizedTensor`` holds its blocks as one
flat byte buffer in ``to_bytes`` order instead of a Vec of enum values.
"""
import ctypes as C
import enum

import numpy as np

from . import _lib
from ._lib import MEM_DEVICE, MEM_HOST, AxqError

DEFAULT_BLOCK_SIZE = 32  # lib.rs:46
MAX_BLOCK_SIZE = 256  # lib.rs:49


# --------------------------------------------------------------------------- errors (error.rs:14-57)
class QuantError(Exception):
    pass


class InvalidBlockSize(QuantError):
    pass


class InvalidQuantType(QuantError):
    pass


class ShapeMismatch(QuantError):
    pass


class DataLengthMismatch(QuantError):
    pass


class CalibrationError(QuantError):
    pass


class Overflow(QuantError):
    pass


class InvalidData(QuantError):
    pass


class TensorConversion(QuantError):
    pass


class DeviceError(QuantError):
    """Device-side failure (CudaError in the reference, backends/cuda.rs:272-289)."""


_STATUS_TO_EXC = {
    -1: InvalidBlockSize, -2: InvalidQuantType, -3: ShapeMismatch, -4: DataLengthMismatch,
    -5: CalibrationError, -6: Overflow, -7: InvalidData, -8: TensorConversion,
}


def _check(lib, ctx_handle, status):
    if status == 0:
        return
    msg = lib.axq_last_error(ctx_handle)
    msg = msg.decode() if msg else lib.axq_status_str(status).decode()
    raise _STATUS_TO_EXC.get(status, DeviceError)(f"{msg} (status {status})")


# --------------------------------------------------------------------------- QuantType (types.rs:17-120)
class QuantType(enum.IntEnum):
    Q8_0 = 0
    Q4_0 = 1
    Q4_1 = 2
    Q5_0 = 3
    Q5_1 = 4
    F16 = 5
    F32 = 6
    Q4_K = 7
    Q6_K = 8
    Q5_K = 9

    def block_size(self):
        return _lib.load_library().axq_type_block_size(int(self))

    def bytes_per_block(self):
        return _lib.load_library().axq_type_bytes_per_block(int(self))

    def bits_per_value(self):
        return _lib.load_library().axq_type_bits_per_value(int(self))

    def compression_ratio(self):
        return 32.0 / self.bits_per_value()

    def is_block_quantized(self):
        return bool(_lib.load_library().axq_type_is_block_quantized(int(self)))

    @staticmethod
    def from_str(s):
        t = _lib.load_library().axq_type_from_str(s.encode())
        return None if t < 0 else QuantType(t)

    def __str__(self):
        return _lib.load_library().axq_type_name(int(self)).decode()


# --------------------------------------------------------------------------- device context
class Context:
    """One GPU, one stream (CudaBackend::new -> Option, backends/cuda.rs:69-81)."""

    def __init__(self, device=0):
        self.lib = _lib.load_library()
        h = C.c_void_p()
        st = self.lib.axq_init(device, C.byref(h))
        if st != 0:
            raise DeviceError(f"{self.lib.axq_last_error(None).decode()} (status {st})")
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.axq_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, status):
        _check(self.lib, self.handle, status)

    def device_info(self):
        info = _lib.DeviceInfo()
        self.check(self.lib.axq_device_info(self.handle, C.byref(info)))
        return info

    def synchronize(self):
        self.check(self.lib.axq_synchronize(self.handle))

    # Backend::allocate / copy_* (backends/mod.rs:73-100)
    def malloc(self, nbytes):
        p = C.c_void_p()
        self.check(self.lib.axq_malloc(self.handle, nbytes, C.byref(p)))
        return p

    def free(self, dptr):
        self.check(self.lib.axq_free(self.handle, dptr))

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.malloc(arr.nbytes)
        self.check(self.lib.axq_copy_to_device(self.handle, p, arr.ctypes.data, arr.nbytes))
        return p

    def to_host(self, dptr, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        self.check(self.lib.axq_copy_to_host(self.handle, out.ctypes.data, dptr, out.nbytes))
        return out

    def timer_start(self):
        self.check(self.lib.axq_timer_start(self.handle))

    def timer_stop(self):
        ms = C.c_float()
        self.check(self.lib.axq_timer_stop(self.handle, C.byref(ms)))
        return ms.value


_default_ctx = None


def default_context():
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context(0)
    return _default_ctx


# --------------------------------------------------------------------------- QuantizedTensor (types.rs:296-334)
class QuantizedTensor:
    """shape, quant_type, blocks (flat ``to_bytes`` image), numel."""

    def __init__(self, shape, quant_type, data):
        self.shape = [int(s) for s in shape]
        self.quant_type = QuantType(quant_type)
        self.numel = int(np.prod(self.shape, dtype=np.int64)) if len(self.shape) else 1
        self.data = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
        expect = _lib.load_library().axq_packed_bytes(int(self.quant_type), self.numel)
        if self.data.size != expect:
            raise DataLengthMismatch(f"Data length mismatch: expected {expect}, got {self.data.size}")

    def num_blocks(self):
        if not self.quant_type.is_block_quantized():
            return 1  # the reference stores F16/F32 as a single block (quantize.rs:215, 226)
        return _lib.load_library().axq_num_blocks(int(self.quant_type), self.numel)

    def size_bytes(self):
        # blocks.len() * bytes_per_block (types.rs:320-322)
        return self.num_blocks() * self.quant_type.bytes_per_block()

    def compression_ratio(self):
        return (self.numel * 4) / float(self.size_bytes())

    def block(self, i):
        bb = self.quant_type.bytes_per_block()
        return self.data[i * bb:(i + 1) * bb]


def _quant_type(v):
    try:
        return QuantType(v)
    except ValueError:
        raise InvalidQuantType(f"Invalid quantization type: {v}")


def quantize_tensor(tensor, quant_type, ctx=None):
    """quantize.rs:36-54: f32 tensor -> QuantizedTensor, blocks along the flat row-major buffer."""
    ctx = ctx or default_context()
    quant_type = _quant_type(quant_type)
    t = np.ascontiguousarray(tensor, dtype=np.float32)
    out = np.empty(ctx.lib.axq_packed_bytes(int(quant_type), t.size), dtype=np.uint8)
    ctx.check(ctx.lib.axq_quantize(ctx.handle, int(quant_type), t.ctypes.data, t.size, out.ctypes.data, MEM_HOST))
    return QuantizedTensor(list(t.shape), quant_type, out)


def quantize_model(tensors, quant_type, ctx=None):
    """quantize.rs:64-75: [(name, tensor)] -> [(name, QuantizedTensor)]; the first error aborts."""
    return [(str(name), quantize_tensor(t, quant_type, ctx)) for name, t in tensors]


def dequantize_tensor(quantized, ctx=None):
    """dequantize.rs:34-54: back to f32 of the original shape (tail block truncated)."""
    ctx = ctx or default_context()
    out = np.empty(quantized.numel, dtype=np.float32)
    ctx.check(ctx.lib.axq_dequantize(ctx.handle, int(quantized.quant_type), quantized.data.ctypes.data,
                                     quantized.numel, out.ctypes.data, MEM_HOST))
    try:
        return out.reshape(quantized.shape)
    except ValueError as e:  # Tensor::from_vec failure (dequantize.rs:52-53)
        raise TensorConversion(str(e))


def dequantize_block(block_bytes, quant_type, ctx=None):
    """dequantize.rs:57-65: one block's byte image -> its block_size floats."""
    ctx = ctx or default_context()
    quant_type = QuantType(quant_type)
    b = np.ascontiguousarray(block_bytes, dtype=np.uint8).reshape(-1)
    if quant_type.is_block_quantized():
        if b.size != quant_type.bytes_per_block():
            raise InvalidData(f"Invalid quantized data: block of {b.size} bytes, expected {quant_type.bytes_per_block()}")
        n = quant_type.block_size()
    else:
        n = b.size // quant_type.bytes_per_block()
    out = np.empty(n, dtype=np.float32)
    ctx.check(ctx.lib.axq_dequantize(ctx.handle, int(quant_type), b.ctypes.data, n, out.ctypes.data, MEM_HOST))
    return out


# --------------------------------------------------------------------------- device weights and matmul
class DeviceWeight:
    """A [n_rows, k] QuantizedTensor resident in HBM."""

    def __init__(self, ctx, handle, quant_type, n_rows, k):
        self.ctx, self.handle = ctx, handle
        self.quant_type, self.n_rows, self.k = QuantType(quant_type), int(n_rows), int(k)

    @classmethod
    def upload(cls, quantized, ctx=None):
        ctx = ctx or default_context()
        if len(quantized.shape) != 2:
            raise ShapeMismatch(f"Shape mismatch: expected a 2-D weight, got {quantized.shape}")
        n, k = quantized.shape
        h = C.c_void_p()
        ctx.check(ctx.lib.axq_weight_upload(ctx.handle, int(quantized.quant_type), n, k, quantized.data.ctypes.data,
                                            quantized.data.size, MEM_HOST, C.byref(h)))
        return cls(ctx, h, quantized.quant_type, n, k)

    @classmethod
    def quantize(cls, weight, quant_type, ctx=None):
        ctx = ctx or default_context()
        w = np.ascontiguousarray(weight, dtype=np.float32)
        if w.ndim != 2:
            raise ShapeMismatch(f"Shape mismatch: expected a 2-D weight, got {list(w.shape)}")
        h = C.c_void_p()
        ctx.check(ctx.lib.axq_weight_quantize(ctx.handle, int(quant_type), w.shape[0], w.shape[1], w.ctypes.data,
                                              MEM_HOST, C.byref(h)))
        return cls(ctx, h, quant_type, w.shape[0], w.shape[1])

    def download(self):
        nbytes = self.ctx.lib.axq_packed_bytes(int(self.quant_type), self.n_rows * self.k)
        out = np.empty(nbytes, dtype=np.uint8)
        self.ctx.check(self.ctx.lib.axq_weight_download(self.ctx.handle, self.handle, out.ctypes.data, nbytes, MEM_HOST))
        return QuantizedTensor([self.n_rows, self.k], self.quant_type, out)

    def free(self):
        if self.handle:
            self.ctx.lib.axq_weight_free(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _as_device_weight(w, ctx):
    if isinstance(w, DeviceWeight):
        return w, False
    return DeviceWeight.upload(w, ctx), True


def quantized_matmul(x, w, bias=None, ctx=None):
    """y = x @ dequantize(w).T (+ bias): Linear::forward (linear.rs:104-140) on packed weights.

    x: f32 [..., k]; w: QuantizedTensor or DeviceWeight of shape [n, k]; returns f32 [..., n].
    """
    ctx = ctx or default_context()
    dw, temp = _as_device_weight(w, ctx)
    try:
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 0 or x.shape[-1] != dw.k:
            raise ShapeMismatch(f"Shape mismatch: expected [..., {dw.k}], got {list(x.shape)}")
        lead = x.shape[:-1]
        batch = int(np.prod(lead, dtype=np.int64)) if lead else 1
        y = np.empty((batch, dw.n_rows), dtype=np.float32)
        b = None
        if bias is not None:
            b = np.ascontiguousarray(bias, dtype=np.float32)
            if b.shape != (dw.n_rows,):
                raise ShapeMismatch(f"Shape mismatch: expected [{dw.n_rows}], got {list(b.shape)}")
        if batch:
            ctx.check(ctx.lib.axq_gemv_f32(ctx.handle, dw.handle, x.ctypes.data, batch,
                                           b.ctypes.data if b is not None else None, y.ctypes.data, MEM_HOST))
        return y.reshape(*lead, dw.n_rows)
    finally:
        if temp:
            dw.free()


def quantized_matmul_bf16(x_bf16, w, ctx=None):
    """Prefill form: x as raw bf16 bits (uint16) [m, k]; returns f32 [m, n]."""
    ctx = ctx or default_context()
    dw, temp = _as_device_weight(w, ctx)
    try:
        x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
        if x.ndim != 2 or x.shape[1] != dw.k:
            raise ShapeMismatch(f"Shape mismatch: expected [m, {dw.k}], got {list(x.shape)}")
        y = np.empty((x.shape[0], dw.n_rows), dtype=np.float32)
        ctx.check(ctx.lib.axq_gemm_bf16(ctx.handle, dw.handle, x.ctypes.data, x.shape[0], y.ctypes.data, MEM_HOST))
        return y
    finally:
        if temp:
            dw.free()


class QuantizedLinear:
    """Linear::from_weights (linear.rs:80-90) over a quantized, device-resident weight."""

    def __init__(self, weight, bias=None, ctx=None):
        self.ctx = ctx or default_context()
        self.weight = weight if isinstance(weight, DeviceWeight) else DeviceWeight.upload(weight, self.ctx)
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self.in_features, self.out_features = self.weight.k, self.weight.n_rows

    def forward(self, x):
        return quantized_matmul(x, self.weight, self.bias, self.ctx)

    __call__ = forward


# --------------------------------------------------------------------------- diagnostics (quantize.rs:235-284)
def compute_quantization_error(original, dequantized):
    """RMSE in f32 (inf when the lengths differ or are zero)."""
    a = np.asarray(original, dtype=np.float32).reshape(-1)
    b = np.asarray(dequantized, dtype=np.float32).reshape(-1)
    if a.size != b.size or a.size == 0:
        return float("inf")
    d = a - b
    return float(np.sqrt(np.float32(np.sum(d * d, dtype=np.float32)) / np.float32(a.size)))


class QuantizationStats:
    """rmse, max_error, mean_error, compression_ratio (quantize.rs:251-261)."""

    def __init__(self, rmse, max_error, mean_error, compression_ratio):
        self.rmse, self.max_error, self.mean_error, self.compression_ratio = rmse, max_error, mean_error, compression_ratio


def compute_quantization_stats(original, dequantized, quant_type):
    """quantize.rs:264-284: error statistics in f32 over the zipped pairs."""
    a = np.asarray(original, dtype=np.float32).reshape(-1)
    b = np.asarray(dequantized, dtype=np.float32).reshape(-1)
    n = min(a.size, b.size)
    err = np.abs(a[:n] - b[:n])
    cnt = np.float32(n)
    with np.errstate(divide="ignore", invalid="ignore"):
        mse = np.sum(err * err, dtype=np.float32) / cnt
        mean = np.sum(err, dtype=np.float32) / cnt
    return QuantizationStats(float(np.sqrt(mse)), float(err.max()) if n else 0.0, float(mean),
                             QuantType(quant_type).compression_ratio())


def f32_to_bf16_bits(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = u + (0x7FFF + ((u >> 16) & 1))
    return (r >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
