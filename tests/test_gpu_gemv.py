"""GPU parity: the decode-path quantized matmul against the CPU oracle.

Bar (north star): max relative error <= 1e-3 against the reference f32 result (accumulation order
differs), relative error taken against max(|ref_i|, 1e-2 * max|ref|); the same 1e-3 against the float64
product of the dequantised weights with the floor at 1e-3 * max|ref|; plus the reference GPU harness's
own |a-b| <= atol + rtol|b| form (backends/gpu_tests.rs:221-249) with rtol = 1e-3."""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from tests.util import MATMUL_RTOL, STRICT_FLOOR, assert_close_ref_style, gen_weight, max_rel_err

pytestmark = pytest.mark.gpu

ALL = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K, o.F16, o.F32]


def _check(ctx, qtype, n, k, batch, seed, outlier_p=0.0, bias=False):
    rng = np.random.default_rng(seed)
    w = gen_weight(rng, n, k, outlier_p=outlier_p)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32) if bias else None
    wq = o.quantize(qtype, w)
    want = o.matmul_ref(qtype, wq, x, n, k, b)
    got = q.quantized_matmul(x, q.QuantizedTensor([n, k], qtype, wq), b, ctx)
    assert got.shape == (batch, n)
    err = max_rel_err(got, want)
    assert err <= MATMUL_RTOL, f"{o.TYPE_NAMES[qtype]} [{n},{k}] b={batch}: max rel err {err:.3e}"
    exact = o.matmul_f64(o.dequantize(qtype, wq, n * k).reshape(n, k), x, b)
    err64 = max_rel_err(got, exact, STRICT_FLOOR)
    assert err64 <= MATMUL_RTOL, f"{o.TYPE_NAMES[qtype]} [{n},{k}] b={batch}: vs float64 {err64:.3e}"
    assert_close_ref_style(got, want, atol=1e-5 * float(np.abs(want).max()), rtol=MATMUL_RTOL)
    return got, want


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("n,k", [(1, 256), (5, 256), (64, 512), (33, 2048), (17, 4096), (130, 4096 + 512),
                                  (9, 11008), (12, 14336), (4, 32768 + 2048)])
def test_gemv_small_shapes(ctx, qtype, n, k):
    if qtype in (o.Q4_K, o.Q5_K, o.Q6_K) and k % 256:
        pytest.skip("k must be a multiple of 256 for the superblock types")
    _check(ctx, qtype, n, k, 1, seed=n * 7 + k)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_1, o.Q8_0, o.Q4_K])
@pytest.mark.parametrize("batch", [2, 8])
def test_gemv_batched_with_bias(ctx, qtype, batch):
    _check(ctx, qtype, 96, 4096, batch, seed=batch, bias=True)


def test_config_q8_0_4096x4096(ctx):
    _check(ctx, o.Q8_0, 4096, 4096, 1, seed=1)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1])
@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("batch", [1, 8])
def test_config_q4_0_q4_1(ctx, qtype, n, k, batch):
    _check(ctx, qtype, n, k, batch, seed=2)


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_config_q4_k_headline(ctx, n, k):
    _check(ctx, o.Q4_K, n, k, 1, seed=3, outlier_p=0.01)


@pytest.mark.parametrize("qtype,n,k", [
    (o.Q4_K, 7001, 2304),   # per-round headers, K slices 1024 + 1024 + 256, rows that do not fill the last workgroup
    (o.Q4_K, 9000, 1280),   # four row groups of three steps: the three-deep ring
    (o.Q4_K, 40000, 1024),  # one slice, eight row groups, two rounds of steps
    (o.Q4_K, 3000, 6144),   # six slices, one row group: per-wave staging, headers per round
    (o.Q4_0, 6000, 320),    # 20 bytes of scales per row: no 16-byte scale loads, the kernel without rounds
    (o.Q4_0, 6000, 1280),   # scales per round, last slice a quarter full
    (o.Q4_1, 5000, 2304),   # two scale loads per round
    (o.Q5_0, 5000, 1536),
    (o.Q5_1, 5000, 1088),   # 136 bytes of scale records per row: the kernel without rounds
    (o.Q8_0, 5000, 2560),
    (o.Q5_K, 7001, 2304),   # the fifth bits come with the headers once per round; last slice a quarter full
    (o.Q5_K, 9000, 1280),
    (o.Q5_K, 3000, 6144),
    (o.Q5_K, 2000, 9216 + 256),  # beyond eight slices: per-wave staging, 37 superblocks
    (o.Q6_K, 7001, 2304),   # bit pairs handed from lane to lane; pieces past the end of a last slice that is not whole
    (o.Q6_K, 9000, 1280),
    (o.Q6_K, 40000, 1024),
    (o.Q6_K, 3000, 6144),
    (o.Q6_K, 5000, 768),    # three superblocks: the second piece of most lanes lies past the row's end
    (o.Q6_K, 2000, 9216 + 256),
])
def test_gemv_scale_records_per_round(ctx, qtype, n, k):
    """Shapes that take the one-vector kernels through several rounds of row steps, partial K slices and ragged row counts."""
    _check(ctx, qtype, n, k, 1, seed=n + k)


@pytest.mark.parametrize("qtype", ALL)
def test_one_hot_activation_selects_dequantised_column(ctx, qtype):
    # exactness of the in-register unpack: y = W[:, col] up to the scale factorisation's rounding
    rng = np.random.default_rng(21)
    n, k = 40, 1024
    w = gen_weight(rng, n, k)
    wq = o.quantize(qtype, w)
    wd = o.dequantize(qtype, wq, n * k).reshape(n, k)
    qt = q.QuantizedTensor([n, k], qtype, wq)
    dw = q.DeviceWeight.upload(qt, ctx)
    for col in (0, 1, 15, 16, 31, 32, 63, 64, 255, 256, 511, 1023):
        x = np.zeros((1, k), np.float32)
        x[0, col] = 1.0
        y = q.quantized_matmul(x, dw, None, ctx)[0]
        assert np.allclose(y, wd[:, col], rtol=1e-5, atol=1e-6 * float(np.abs(wd).max())), (o.TYPE_NAMES[qtype], col)
    dw.free()


def test_linearity_and_determinism_at_full_size(ctx):
    rng = np.random.default_rng(8)
    n, k = 4096, 14336
    dw = q.DeviceWeight.quantize(gen_weight(rng, n, k, outlier_p=0.01), q.QuantType.Q4_K, ctx)
    x1 = rng.standard_normal((1, k)).astype(np.float32)
    x2 = rng.standard_normal((1, k)).astype(np.float32)
    y1 = q.quantized_matmul(x1, dw, None, ctx)
    y2 = q.quantized_matmul(x2, dw, None, ctx)
    y12 = q.quantized_matmul(x1 + 2 * x2, dw, None, ctx)
    assert max_rel_err(y12, y1.astype(np.float64) + 2 * y2.astype(np.float64)) < 1e-4
    assert np.array_equal(q.quantized_matmul(x1, dw, None, ctx), y1)  # no atomics: run-to-run identical
    dw.free()


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q6_K, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0])
@pytest.mark.parametrize("k", [512, 4096, 32768 + 256])
def test_activations_with_a_mean_do_not_cancel(ctx, qtype, k):
    # post-softmax / post-SiLU activations are not zero-mean: offsets of the unsigned codes must be
    # removed exactly, not by subtracting two large f32 sums.  Checked against the float64 product
    # at the strict floor for a positive-mean, a tiny and a spiky input.
    rng = np.random.default_rng(k + qtype)
    n = 64
    w = gen_weight(rng, n, k, std=0.06)
    wq = o.quantize(qtype, w)
    wd = o.dequantize(qtype, wq, n * k).reshape(n, k)
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
    for x in (0.3 + 0.05 * rng.standard_normal((1, k)), 1e-3 * rng.standard_normal((1, k)),
              rng.standard_normal((1, k)) * np.where(np.arange(k) % 32 < 4, 10.0, 0.01)):
        x = x.astype(np.float32)
        got = q.quantized_matmul(x, dw, None, ctx)
        assert max_rel_err(got, o.matmul_f64(wd, x), STRICT_FLOOR) <= 2e-4
    dw.free()


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q6_K, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0])
@pytest.mark.parametrize("batch,n,k", [(8, 520, 4096), (3, 264, 14336)])
def test_small_batch_activations_with_a_mean_do_not_cancel(ctx, qtype, batch, n, k):
    """The same for the small-batch kernel: rows on an offset of 20 standard deviations, all positive, or negative.  Its
    codes go into the matrix pipe centred; as unsigned codes with the offset in a separate sum over x these rows came out
    at 4-8e-4 at the strict floor."""
    rng = np.random.default_rng(batch + n + k + qtype)
    wq = o.quantize(qtype, gen_weight(rng, n, k))
    wd = o.dequantize(qtype, wq, n * k).reshape(n, k)
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    x[0] = 1.0 + 0.05 * x[0]
    x[1] = 10.0 + x[1]
    x[2] = -3.0 + 0.1 * x[2]
    got = q.quantized_matmul(x, dw, None, ctx)
    exact = o.matmul_f64(wd, x)
    for r in range(batch):
        assert max_rel_err(got[r], exact[r], STRICT_FLOOR) <= 3e-4, r
    dw.free()


def test_quantized_linear_keeps_leading_dims(ctx):
    rng = np.random.default_rng(4)
    w = gen_weight(rng, 48, 512)
    lin = q.QuantizedLinear(q.quantize_tensor(w, q.QuantType.Q4_1, ctx), rng.standard_normal(48).astype(np.float32), ctx)
    x = rng.standard_normal((2, 3, 512)).astype(np.float32)
    y = lin(x)
    assert y.shape == (2, 3, 48)
    want = o.matmul_ref(o.Q4_1, o.quantize(o.Q4_1, w), x.reshape(6, 512), 48, 512, lin.bias).reshape(2, 3, 48)
    assert max_rel_err(y, want) <= MATMUL_RTOL


def test_gemv_shape_errors(ctx):
    w = q.quantize_tensor(np.zeros((4, 256), np.float32), q.QuantType.Q8_0, ctx)
    with pytest.raises(q.ShapeMismatch):
        q.quantized_matmul(np.zeros((1, 128), np.float32), w, None, ctx)
    with pytest.raises(q.ShapeMismatch):
        q.quantized_matmul(np.zeros((1, 256), np.float32), w, np.zeros(3, np.float32), ctx)


# ---- small batches: one pass over the weights for up to eight vectors (v_mfma_i32_32x32x32_i8 path)
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q4_K, o.Q5_K, o.Q6_K])
@pytest.mark.parametrize("batch,n,k", [(2, 32, 512), (3, 100, 1024), (8, 96, 4096), (8, 33, 512), (11, 64, 2048), (16, 40, 4096),
                                       (2, 32, 256), (8, 33, 768), (8, 40, 11008), (5, 64, 14336), (8, 32, 16384)])
def test_small_batch_reads_weights_once(ctx, qtype, batch, n, k):
    rng = np.random.default_rng(batch * 1000 + n + k + qtype)
    w = gen_weight(rng, n, k)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    x[1] = 0.3 + 0.05 * x[1]  # one vector with a mean: code offsets must cancel exactly for it too
    bias = rng.standard_normal(n).astype(np.float32)
    wq = o.quantize(qtype, w)
    want = o.matmul_ref(qtype, wq, x, n, k, bias)
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
    got = q.quantized_matmul(x, dw, bias, ctx)
    assert got.shape == (batch, n)
    assert max_rel_err(got, want) <= MATMUL_RTOL
    exact = o.matmul_f64(o.dequantize(qtype, wq, n * k).reshape(n, k), x) + bias.astype(np.float64)
    assert max_rel_err(got, exact, STRICT_FLOOR) <= MATMUL_RTOL
    # the batched kernel and the one-vector kernel agree far inside the tolerance
    one = np.stack([q.quantized_matmul(x[i:i + 1], dw, bias, ctx)[0] for i in range(batch)])
    assert max_rel_err(got, one, STRICT_FLOOR) <= 3e-4  # f32 summation orders differ; at this floor that is the noise
    dw.free()


# ---- many vectors: f32 rows through the matrix-pipe GEMM as two f16 rows each
@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q6_K, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.F16, o.F32])
@pytest.mark.parametrize("batch,n,k", [(40, 96, 512), (64, 100, 1024), (130, 33, 4096), (9, 64, 2048), (300, 257, 768), (384, 132, 512),
                                       (777, 64, 1024)])
def test_many_vectors_go_through_the_gemm_at_f32_accuracy(ctx, qtype, batch, n, k):
    rng = np.random.default_rng(batch * 7 + n + k + qtype)
    w = gen_weight(rng, n, k)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    x[1] = 0.3 + 0.05 * x[1]
    x[2] *= 1e-3                      # rows of very different magnitude: every row has its own scale
    x[3, ::7] *= 1e-4                 # small elements beside large ones inside a row
    x[4] *= 3e4
    bias = rng.standard_normal(n).astype(np.float32)
    wq = o.quantize(qtype, w)
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
    got = q.quantized_matmul(x, dw, bias, ctx)
    assert got.shape == (batch, n)
    exact = o.matmul_f64(o.dequantize(qtype, wq, n * k).reshape(n, k), x) + bias.astype(np.float64)
    # row by row, so that the large rows do not hide the small ones
    for r in range(batch):
        assert max_rel_err(got[r], exact[r], STRICT_FLOOR) <= MATMUL_RTOL, r
    # far inside the tolerance: the split of a row into two f16 rows keeps 22 bits
    rel = np.abs(got - exact).max(axis=1) / np.abs(exact).max(axis=1)
    assert rel.max() <= 2e-5, rel.max()
    dw.free()


@pytest.mark.parametrize("batch", [48, 400])
def test_many_vectors_non_finite_row(ctx, batch):
    rng = np.random.default_rng(5)
    n, k = 64, 512
    wq = o.quantize(o.Q4_K, gen_weight(rng, n, k))
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], o.Q4_K, wq), ctx)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    x[5, 100] = np.nan
    x[7, 3] = np.inf
    y = q.quantized_matmul(x, dw, None, ctx)
    assert not np.isfinite(y[5]).any() and not np.isfinite(y[7]).any()
    keep = [r for r in range(batch) if r not in (5, 7)]
    assert np.isfinite(y[keep]).all()
    dw.free()


@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 11008)])
def test_small_batch_config_shape(ctx, n, k):
    # the 7B LLaMA feed-forward shapes: 11008 x 4096 and the transposed down-projection, batch 8, Q4_0 and Q4_1
    rng = np.random.default_rng(82)
    batch = 8
    w = gen_weight(rng, n, k)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    for qtype in (o.Q4_0, o.Q4_1):
        wq = o.quantize(qtype, w)
        dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
        got = q.quantized_matmul(x, dw, None, ctx)
        exact = o.matmul_f64(o.dequantize(qtype, wq, n * k).reshape(n, k), x)
        assert max_rel_err(got, exact, STRICT_FLOOR) <= MATMUL_RTOL
        dw.free()


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("batch", [1, 8])
def test_non_finite_activation_reaches_every_output(ctx, qtype, batch):
    # a nan (or an infinity) in x makes every f32 dot product of the reference non-finite; the integer limb
    # split must not lose it (a float maximum ignores nan operands)
    rng = np.random.default_rng(17)
    n, k = 64, 4096
    dw = q.DeviceWeight.quantize(gen_weight(rng, n, k), q.QuantType(qtype), ctx)
    for bad in (np.nan, np.inf, -np.inf):
        x = rng.standard_normal((batch, k)).astype(np.float32)
        x[0, 1234] = bad
        y = q.quantized_matmul(x, dw, None, ctx)
        assert not np.isfinite(y[0]).any(), (o.TYPE_NAMES[qtype], bad)
        if np.isnan(bad):
            assert np.isnan(y[0]).all()
        if batch > 1:
            assert np.isfinite(y[1:]).all()  # the other vectors of the batch are untouched
    dw.free()
