"""GPU parity: the prefill-path quantized GEMM (bf16 activations, f32 accumulate) against the CPU oracle.

Bar: max relative error <= 1e-3 against the reference f32 result (dequantise -> f32 sgemm on the same
bf16 inputs widened exactly), relative error taken against max(|ref_i|, 1e-2 * max|ref|), and the same
bound against the float64 product at the 1e-3 floor."""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from tests.util import MATMUL_RTOL, STRICT_FLOOR, gen_weight, max_rel_err

pytestmark = pytest.mark.gpu

ALL = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K, o.F16, o.F32]


def _check(ctx, qtype, m, n, k, seed, xscale=1.0):
    rng = np.random.default_rng(seed)
    w = gen_weight(rng, n, k)
    xb = q.f32_to_bf16_bits((rng.standard_normal((m, k)) * xscale).astype(np.float32))
    x = q.bf16_bits_to_f32(xb)
    wq = o.quantize(qtype, w)
    want = o.matmul_ref(qtype, wq, x, n, k)
    got = q.quantized_matmul_bf16(xb, q.QuantizedTensor([n, k], qtype, wq), ctx)
    assert got.shape == (m, n)
    err = max_rel_err(got, want)
    assert err <= MATMUL_RTOL, f"{o.TYPE_NAMES[qtype]} M={m} N={n} K={k}: max rel err {err:.3e}"
    exact = o.matmul_f64(o.dequantize(qtype, wq, n * k).reshape(n, k), x)
    assert max_rel_err(got, exact, STRICT_FLOOR) <= MATMUL_RTOL


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("m,n,k", [(1, 128, 256), (7, 64, 256), (128, 128, 512), (130, 200, 1024), (300, 256, 768)])
def test_gemm_small_shapes(ctx, qtype, m, n, k):
    _check(ctx, qtype, m, n, k, seed=m + n + k + qtype)


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q5_1])
@pytest.mark.parametrize("m", [128, 512])
def test_config_prefill_k4096(ctx, qtype, m):
    _check(ctx, qtype, m, 512, 4096, seed=m)


@pytest.mark.parametrize("qtype", [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K])
@pytest.mark.parametrize("m,n,k", [(250, 300, 1024), (640, 136, 512), (1100, 520, 1024)])
def test_many_rows(ctx, qtype, m, n, k):
    """Several row tiles per column tile, ragged in both directions."""
    _check(ctx, qtype, m, n, k, seed=m + qtype)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_1, o.Q8_0])
@pytest.mark.parametrize("m", [40, 160])
def test_llama_ffn_width_with_an_odd_count_of_superblocks(ctx, qtype, m):
    """K = 11008 (the 7B LLaMA feed-forward width, 43 superblocks of 256): the block-of-32 kernel's two record buffers and
    its split of K over workgroups at an odd count, on both of its row tiles."""
    _check(ctx, qtype, m, 96, 11008, seed=m + qtype)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0])
@pytest.mark.parametrize("m,n,k", [(1, 1, 256), (127, 31, 768), (129, 129, 256), (257, 255, 512), (300, 130, 2304), (513, 4, 1280)])
def test_ragged_tiles_of_the_block_of_32_kernel(ctx, qtype, m, n, k):
    """Row and column counts on both sides of its tile edges (128 and 256 rows, 128 columns, 32 and 64 per wave), one
    superblock and an odd count of them, every type it takes."""
    _check(ctx, qtype, m, n, k, seed=m * 3 + n + k + qtype)


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K])
@pytest.mark.parametrize("m,n,k", [(1, 1, 256), (127, 31, 768), (129, 129, 256), (257, 255, 512), (300, 130, 2304), (513, 4, 1280),
                                   (260, 520, 4352)])
def test_ragged_tiles_of_the_superblock_kernel(ctx, qtype, m, n, k):
    """Row and column counts on both sides of its tile edges (128 and 256 rows, 256 columns, 64 per wave), one superblock,
    odd counts of them (the minimum term takes them in pairs) and a K that is split over workgroups unevenly; Q5_K's fifth
    bits ride along with the codes."""
    _check(ctx, qtype, m, n, k, seed=m * 3 + n + k + qtype)


@pytest.mark.parametrize("qtype", [o.Q4_1, o.Q5_1, o.Q4_0, o.Q5_0, o.Q8_0, o.Q4_K, o.Q5_K, o.Q6_K])
@pytest.mark.parametrize("m", [48, 300])
def test_large_weights_block_minimums_beyond_256_and_scales_beyond_32(ctx, qtype, m):
    """Weights around 300 with a spread of 100: block minimums of magnitude 256 and more, block scales of 16 to 40.  The
    reference's dequantise -> f32 sgemm is finite there, so the GEMM has to be (operands formed as minimum x 256 or
    16 d x 256 in f16 would overflow)."""
    rng = np.random.default_rng(300 + qtype + m)
    n, k = 160, 1024
    w = (gen_weight(rng, n, k) * 5000.0 + 300.0).astype(np.float32)
    xb = q.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    x = q.bf16_bits_to_f32(xb)
    wq = o.quantize(qtype, w)
    deq = o.dequantize(qtype, wq, n * k)
    assert np.abs(deq).max() > 500
    want = o.matmul_ref(qtype, wq, x, n, k)
    got = q.quantized_matmul_bf16(xb, q.QuantizedTensor([n, k], qtype, wq), ctx)
    assert np.isfinite(got).all()
    assert max_rel_err(got, want) <= MATMUL_RTOL
    assert max_rel_err(got, o.matmul_f64(deq.reshape(n, k), x), STRICT_FLOOR) <= MATMUL_RTOL


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K])
@pytest.mark.parametrize("xscale", [1e-30, 1e30])
def test_many_rows_of_extreme_magnitude(ctx, qtype, xscale):
    _check(ctx, qtype, 1030, 128, 512, seed=11, xscale=xscale)


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q4_1, o.Q5_1, o.Q6_K])
@pytest.mark.parametrize("m,n,k", [(130, 33, 4096), (300, 520, 2048)])
def test_activation_rows_with_a_mean(ctx, qtype, m, n, k):
    """Rows that are all positive or sit on an offset: the sums over the codes and over the block minimums are then each
    far larger than the result, and a kernel that adds them separately has to keep their rounding below the bound for
    the row's small outputs too (codes centred before they are summed).  Both entry points, row by row."""
    rng = np.random.default_rng(m + n + k + qtype)
    wq = o.quantize(qtype, gen_weight(rng, n, k))
    deq = o.dequantize(qtype, wq, n * k).reshape(n, k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[1] = 0.3 + 0.05 * x[1]
    x[5] = np.abs(x[5])
    x[6] = 5.0 + x[6]
    x[7] = -2.0 + 0.5 * x[7]
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, wq), ctx)
    xb = q.f32_to_bf16_bits(x)
    for got, xin in ((q.quantized_matmul_bf16(xb, dw, ctx), q.bf16_bits_to_f32(xb)), (q.quantized_matmul(x, dw, None, ctx), x)):
        exact = o.matmul_f64(deq, xin)
        for r in range(m):
            assert max_rel_err(got[r], exact[r], STRICT_FLOOR) <= MATMUL_RTOL, (r, o.TYPE_NAMES[qtype])
    dw.free()


@pytest.mark.parametrize("xscale", [1e-4, 1.0, 3e4])
def test_row_scaling_keeps_extreme_activations_exact(ctx, xscale):
    _check(ctx, o.Q4_K, 64, 128, 512, seed=9, xscale=xscale)


def test_rows_with_different_magnitudes(ctx):
    rng = np.random.default_rng(3)
    m, n, k = 96, 128, 512
    w = gen_weight(rng, n, k)
    x = rng.standard_normal((m, k)).astype(np.float32) * (10.0 ** rng.integers(-6, 6, size=(m, 1))).astype(np.float32)
    xb = q.f32_to_bf16_bits(x)
    x = q.bf16_bits_to_f32(xb)
    wq = o.quantize(o.Q4_K, w)
    want = o.matmul_f64(o.dequantize(o.Q4_K, wq, n * k).reshape(n, k), x)
    got = q.quantized_matmul_bf16(xb, q.QuantizedTensor([n, k], o.Q4_K, wq), ctx)
    for r in range(m):  # per row: each row has its own scale
        assert max_rel_err(got[r], want[r], STRICT_FLOOR) <= MATMUL_RTOL, r


def test_gemm_matches_gemv_path(ctx):
    rng = np.random.default_rng(5)
    n, k = 256, 1024
    dw = q.DeviceWeight.quantize(gen_weight(rng, n, k), q.QuantType.Q4_K, ctx)
    xb = q.f32_to_bf16_bits(rng.standard_normal((4, k)).astype(np.float32))
    y_gemm = q.quantized_matmul_bf16(xb, dw, ctx)
    y_gemv = q.quantized_matmul(q.bf16_bits_to_f32(xb), dw, None, ctx)
    assert max_rel_err(y_gemm, y_gemv) <= 1e-4
    dw.free()


def test_gemm_shape_errors(ctx):
    w = q.quantize_tensor(np.zeros((4, 256), np.float32), q.QuantType.Q8_0, ctx)
    with pytest.raises(q.ShapeMismatch):
        q.quantized_matmul_bf16(np.zeros((2, 128), np.uint16), w, ctx)
    w32 = q.quantize_tensor(np.zeros((4, 96), np.float32), q.QuantType.Q8_0, ctx)
    with pytest.raises(q.InvalidBlockSize):  # the GEMM needs k % 64 == 0
        q.quantized_matmul_bf16(np.zeros((2, 96), np.uint16), w32, ctx)
