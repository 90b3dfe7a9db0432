"""Shared helpers for the parity tests."""
import numpy as np

# The path's matmul tolerance: max relative error 1e-3 against the reference f32 result.  The relative
# error of output i is |y_i - ref_i| / max(|ref_i|, FLOOR * max_j |ref_j|), so that outputs that happen
# to be near zero do not divide by nothing.  Two floors are used:
#   REL_FLOOR = 1e-2 against the f32 oracle (the reference's own result).  A tighter floor would measure
#     the reference's accumulation noise, not the kernel: the oracle's f32 sgemm already sits 9e-4 away
#     from the exact product at a 1e-3 floor for K = 11008 (tests/test_oracle_matmul.py pins that).
#   STRICT_FLOOR = 1e-3 against the float64 product of the same dequantised weights (the exact answer).
MATMUL_RTOL = 1e-3
REL_FLOOR = 1e-2
STRICT_FLOOR = 1e-3
# Logits after a whole decoder stack are compared normwise: max|y - ref| / max|ref| <= 1e-3 (DECODE_FLOOR = 1
# in max_rel_err).  The per-element floor metric is the wrong instrument there, because rounding k and v to
# f16 for the cache is a discontinuity: two correct f32 evaluations that differ in the last bits upstream
# round an occasional cache element to neighbouring f16 values (tests/test_gpu_decode.py counts them: a few
# per thousand, one f16 ulp each), and each such flip moves every logit by ~1e-5 of the logit range --
# invisible normwise (measured 6e-5), but several 1e-3 of a logit that happens to be near zero.
DECODE_RTOL = 1e-3
DECODE_FLOOR = 1.0


def max_rel_err(got, want, floor=REL_FLOOR):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    denom = np.maximum(np.abs(want), floor * np.abs(want).max())
    denom = np.where(denom == 0, 1.0, denom)
    return float((np.abs(got - want) / denom).max())


def assert_close_ref_style(got, want, atol=1e-5, rtol=1e-3):
    """The reference GPU harness's check: |a - b| <= atol + rtol * |b| (backends/gpu_tests.rs:221-249)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    bad = np.abs(got - want) > atol + rtol * np.abs(want)
    assert not bad.any(), f"{int(bad.sum())} of {bad.size} outside atol={atol} rtol={rtol}"


def gen_weight(rng, n, k, std=0.02, outlier_p=0.0, outlier_mag=0.5):
    w = (rng.standard_normal((n, k)) * std).astype(np.float32)
    if outlier_p > 0:
        mask = rng.random((n, k)) < outlier_p
        sign = np.where(rng.random((n, k)) < 0.5, -1.0, 1.0).astype(np.float32)
        w = np.where(mask, sign * np.float32(outlier_mag), w).astype(np.float32)
    return w
