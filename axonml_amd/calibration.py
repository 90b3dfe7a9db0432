"""Host-side mirror of the reference's calibration statistics (crates/axonml-quant/src/calibration.rs:19-232).

In the reference these statistics are bookkeeping next to the quantisers, not an input to them: every block
codec derives its own scale from the block (quantize.rs:94-100, 139, 175-179).  They are plain f32 reductions
over a tensor on the host, kept here with the same names, fields and results so that callers of the crate find
them; nothing on the device path depends on them."""
import enum

import numpy as np

from .quant import CalibrationError, QuantType

_F = np.float32


def _flat(t):
    return np.ascontiguousarray(t, dtype=np.float32).reshape(-1)


class CalibrationData:
    """min, max, mean, std_dev, num_samples and a histogram (calibration.rs:19-66)."""

    def __init__(self, tensor, num_bins):
        d = _flat(tensor)
        self.min = float(d.min()) if d.size else float("inf")
        self.max = float(d.max()) if d.size else float("-inf")
        n = _F(d.size)
        self.mean = float(np.sum(d, dtype=np.float32) / n)
        var = np.sum((d - _F(self.mean)) ** 2, dtype=np.float32) / n
        self.std_dev = float(np.sqrt(var))
        self.num_samples = int(d.size)
        width = (_F(self.max) - _F(self.min)) / _F(num_bins)
        self._bin_edges = (_F(self.min) + np.arange(num_bins + 1, dtype=np.float32) * width).astype(np.float32)
        with np.errstate(divide="ignore", invalid="ignore"):
            idx = ((d - _F(self.min)) / width)
        idx = np.where(np.isfinite(idx), idx, 0).astype(np.int64)  # `as usize` saturates; nan -> 0
        idx = np.clip(idx, 0, num_bins - 1)
        self._histogram = np.bincount(idx, minlength=num_bins)

    def update(self, tensor):
        """calibration.rs:69-85: widens min/max and merges the mean; the histogram and std_dev stay as they were."""
        d = _flat(tensor)
        self.min = min(self.min, float(d.min()))
        self.max = max(self.max, float(d.max()))
        old, new = _F(self.num_samples), _F(d.size)
        new_mean = np.sum(d, dtype=np.float32) / new
        self.mean = float((_F(self.mean) * old + new_mean * new) / (old + new))
        self.num_samples += int(d.size)

    def dynamic_range(self):
        return float(_F(self.max) - _F(self.min))

    def symmetric_scale(self, quant_type):
        """max(|min|, |max|) / largest code (calibration.rs:93-102)."""
        max_int = {QuantType.Q8_0: 127.0, QuantType.Q4_0: 7.0, QuantType.Q4_1: 7.0, QuantType.Q4_K: 7.0, QuantType.Q6_K: 31.0, QuantType.Q5_K: 15.0,
                   QuantType.Q5_0: 15.0, QuantType.Q5_1: 15.0, QuantType.F16: 1.0, QuantType.F32: 1.0}[QuantType(quant_type)]
        return float(_F(max(abs(self.min), abs(self.max))) / _F(max_int))

    def asymmetric_scale(self, quant_type):
        """(scale, zero_point) over the full unsigned code range (calibration.rs:105-117)."""
        max_int = {QuantType.Q8_0: 255.0, QuantType.Q4_0: 15.0, QuantType.Q4_1: 15.0, QuantType.Q4_K: 15.0, QuantType.Q6_K: 63.0, QuantType.Q5_K: 31.0,
                   QuantType.Q5_0: 31.0, QuantType.Q5_1: 31.0, QuantType.F16: 1.0, QuantType.F32: 1.0}[QuantType(quant_type)]
        scale = (_F(self.max) - _F(self.min)) / _F(max_int)
        with np.errstate(divide="ignore", invalid="ignore"):
            zero_point = -_F(self.min) / scale
        return float(scale), float(zero_point)

    def percentile(self, p):
        """Left edge of the first bin at which the cumulative count reaches p % (calibration.rs:120-140)."""
        if p <= 0.0:
            return self.min
        if p >= 100.0:
            return self.max
        target = int(_F(p) / _F(100.0) * _F(self.num_samples))
        cum = np.cumsum(self._histogram)
        hit = np.nonzero(cum >= target)[0]
        return float(self._bin_edges[hit[0]]) if hit.size else self.max


class CalibrationMethod(enum.Enum):
    """calibration.rs:148-158.  Percentile and MeanStd carry their parameter times ten (999 = 99.9 %, 30 = 3 sigma)."""
    MinMax = "minmax"
    Percentile = "percentile"
    Entropy = "entropy"
    MeanStd = "meanstd"


def _clip(data, method, param):
    if method is CalibrationMethod.Percentile:
        p = _F(param) / _F(10.0)
        lower, upper = data.percentile(float(_F(100.0) - p)), data.percentile(float(p))
        data.min, data.max = lower, upper
    elif method is CalibrationMethod.MeanStd:
        k = _F(param) / _F(10.0)
        data.min = float(_F(data.mean) - k * _F(data.std_dev))
        data.max = float(_F(data.mean) + k * _F(data.std_dev))


def calibrate(tensor, method=CalibrationMethod.MinMax, param=None):
    """calibration.rs:161-191 (2048 bins)."""
    data = CalibrationData(tensor, 2048)
    if method is CalibrationMethod.Entropy:
        data.min, data.max = data.percentile(0.01), data.percentile(99.99)
    else:
        _clip(data, method, param)
    return data


def calibrate_batch(tensors, method=CalibrationMethod.MinMax, param=None):
    """calibration.rs:194-232: statistics of the first tensor, widened by the others."""
    tensors = list(tensors)
    if not tensors:
        raise CalibrationError("Calibration error: No tensors provided")
    combined = CalibrationData(tensors[0], 2048)
    for t in tensors[1:]:
        combined.update(t)
    _clip(combined, method, param)  # MinMax and Entropy leave the range as it is here, as in the reference
    return combined
