"""Host-side statistics mirrors: the reference's own calibration tests (calibration.rs:242-291) and the
quantisation-error helpers (quantize.rs:235-284), restated."""
import numpy as np
import pytest

from axonml_amd import quant as q
from axonml_amd.calibration import CalibrationData, CalibrationMethod, calibrate, calibrate_batch


def test_calibration_data():  # calibration.rs:243-253
    c = CalibrationData(np.array([1.0, 2.0, 3.0, 4.0, 5.0], np.float32), 10)
    assert (c.min, c.max, c.mean, c.num_samples) == (1.0, 5.0, 3.0, 5)
    assert abs(c.std_dev - np.sqrt(2.0)) < 1e-6


def test_symmetric_scale():  # calibration.rs:255-265
    c = CalibrationData(np.array([-4.0, -2.0, 0.0, 2.0, 4.0], np.float32), 10)
    assert abs(c.symmetric_scale(q.QuantType.Q8_0) - 4.0 / 127.0) < 0.001
    scale, zp = c.asymmetric_scale(q.QuantType.Q4_1)
    assert abs(scale - 8.0 / 15.0) < 1e-6 and abs(zp - 7.5) < 1e-5


def test_calibration_methods():  # calibration.rs:267-281
    t = (np.arange(1000) / 100.0).astype(np.float32)
    mm = calibrate(t, CalibrationMethod.MinMax)
    assert abs(mm.min - 0.0) < 0.01 and abs(mm.max - 9.99) < 0.01
    p = calibrate(t, CalibrationMethod.Percentile, 999)
    assert p.min >= 0.0 and p.max <= 9.99
    ms = calibrate(t, CalibrationMethod.MeanStd, 30)
    assert abs(ms.min - (ms.mean - 3 * ms.std_dev)) < 1e-4 and abs(ms.max - (ms.mean + 3 * ms.std_dev)) < 1e-4
    e = calibrate(t, CalibrationMethod.Entropy)
    assert 0.0 <= e.min <= 0.01 and 9.9 <= e.max <= 9.99


def test_dynamic_range():  # calibration.rs:283-290
    assert CalibrationData(np.array([-5.0, 10.0], np.float32), 10).dynamic_range() == 15.0


def test_percentile_walks_the_histogram():
    c = CalibrationData(np.arange(100, dtype=np.float32), 10)  # ten bins of ten samples, edges 0, 9.9, 19.8, ...
    assert c.percentile(0.0) == 0.0 and c.percentile(100.0) == 99.0
    assert c.percentile(10.0) == 0.0          # the first bin already holds ten samples
    assert abs(c.percentile(50.0) - 39.6) < 1e-4


def test_calibrate_batch():
    with pytest.raises(q.CalibrationError):
        calibrate_batch([])
    a, b = np.array([0.0, 1.0, 2.0, 3.0], np.float32), np.array([-2.0, 10.0], np.float32)
    c = calibrate_batch([a, b])
    assert (c.min, c.max, c.num_samples) == (-2.0, 10.0, 6)
    assert abs(c.mean - (1.5 * 4 + 4.0 * 2) / 6) < 1e-6


def test_quantization_error_helpers():  # quantize.rs:235-284
    a = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    b = np.array([1.5, 2.0, 2.0, 4.0], np.float32)
    assert abs(q.compute_quantization_error(a, b) - np.sqrt((0.25 + 1.0) / 4)) < 1e-6
    assert q.compute_quantization_error(a, b[:3]) == float("inf") and q.compute_quantization_error([], []) == float("inf")
    s = q.compute_quantization_stats(a, b, q.QuantType.Q4_0)
    assert abs(s.rmse - np.sqrt(1.25 / 4)) < 1e-6 and s.max_error == 1.0 and abs(s.mean_error - 0.375) < 1e-6
    assert s.compression_ratio == 8.0
