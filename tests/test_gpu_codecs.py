"""GPU parity: device quantize / dequantize / weight upload-download against the CPU oracle.

Bar: bit-exact packed bytes (codes and f16 scales) and bit-exact dequantised f32."""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from tests.util import gen_weight

pytestmark = pytest.mark.gpu

ALL = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K, o.F16, o.F32]
BLOCK = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K]
SUPER = (o.Q4_K, o.Q5_K, o.Q6_K)  # 256-element superblocks


def _inputs(rng, n):
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x[rng.random(n) < 0.01] = 0.5
    x[rng.random(n) < 0.01] = -0.5
    return x


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("n", [1, 31, 32, 33, 35, 40, 255, 256, 257, 4096, 100003])
def test_quantize_bit_exact(ctx, qtype, n):
    x = _inputs(np.random.default_rng(100 + n), n)
    got = q.quantize_tensor(x, qtype, ctx)
    want = o.quantize(qtype, x)
    assert got.data.size == want.size
    bad = np.nonzero(got.data != want)[0]
    assert bad.size == 0, f"{o.TYPE_NAMES[qtype]} n={n}: {bad.size} bytes differ, first at {bad[0]}"


@pytest.mark.parametrize("qtype", BLOCK)
def test_quantize_special_blocks_bit_exact(ctx, qtype):
    bs = 256 if qtype in SUPER else 32
    blocks = [
        np.zeros(bs), np.full(bs, 2.5), np.full(bs, -2.5), np.arange(bs) - bs / 2, np.arange(bs) / 10.0,
        np.where(np.arange(bs) % 2 == 0, 0.5, -0.5) * np.arange(bs),  # many exact half-way quotients
        np.r_[127.0, -127.0, 0.5, -0.5, 1.5, 2.5, -2.5, np.zeros(bs - 7)],
        np.r_[7.0, -7.0, 6.5, -6.5, 0.5, -0.5, 2.5, np.zeros(bs - 7)],
        np.r_[0.0, 15.0, 0.5, 1.5, 2.5, 14.5, np.zeros(bs - 6)],
        np.r_[0.0, 31.0, 0.5, 1.5, 2.5, 30.5, np.zeros(bs - 6)],
        np.r_[1e-30, -1e-30, np.zeros(bs - 2)], np.r_[6e4, -6e4, 1e5, np.zeros(bs - 3)],
        np.full(bs, 1e-8), -np.abs(np.arange(bs) - 5.0),
    ]
    x = np.concatenate(blocks).astype(np.float32)
    got = q.quantize_tensor(x, qtype, ctx)
    assert np.array_equal(got.data, o.quantize(qtype, x))


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("n", [1, 33, 40, 256, 300, 8192, 100003])
def test_dequantize_bit_exact(ctx, qtype, n):
    x = _inputs(np.random.default_rng(200 + n), n)
    packed = o.quantize(qtype, x)
    qt = q.QuantizedTensor([n], qtype, packed)
    got = q.dequantize_tensor(qt, ctx)
    want = o.dequantize(qtype, packed, n)
    assert got.shape == (n,)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype", BLOCK)
def test_dequantize_arbitrary_bytes_bit_exact(ctx, qtype):
    # every code/bit pattern, not only what the quantiser emits (scales kept finite)
    rng = np.random.default_rng(77)
    bb = o.lib().axo_bytes_per_block(qtype)
    nblk = 512
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    nscale = {o.Q8_0: 1, o.Q4_0: 1, o.Q5_0: 1, o.Q4_1: 2, o.Q5_1: 2, o.Q4_K: 2, o.Q5_K: 2, o.Q6_K: 1}[qtype]
    scales = (rng.standard_normal((nblk, nscale)) * 0.1).astype(np.float16)
    at = 208 if qtype == o.Q6_K else 0  # Q6_K keeps its f16 d behind the codes and the int8 scales (all 256 values occur)
    raw[:, at:at + 2 * nscale] = scales.view(np.uint8)
    n = nblk * (256 if qtype in SUPER else 32)
    got = q.dequantize_tensor(q.QuantizedTensor([n], qtype, raw.reshape(-1)), ctx)
    want = o.dequantize(qtype, raw.reshape(-1), n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_reference_roundtrip_cases_on_device(ctx):
    # dequantize.rs:204-272 through the device codecs
    x = np.arange(64, dtype=np.float32) / np.float32(10.0)
    y8 = q.dequantize_tensor(q.quantize_tensor(x, q.QuantType.Q8_0, ctx), ctx)
    assert y8.shape == (64,) and np.abs(y8 - x).max() < 0.1
    y4 = q.dequantize_tensor(q.quantize_tensor(x, q.QuantType.Q4_0, ctx), ctx)
    assert np.abs(y4 - x).max() < 2.0
    v = np.array([1.0, 2.5, -3.0, 4.25], np.float32)
    assert np.abs(q.dequantize_tensor(q.quantize_tensor(v, q.QuantType.F16, ctx), ctx) - v).max() < 0.01
    assert np.array_equal(q.dequantize_tensor(q.quantize_tensor(v, q.QuantType.F32, ctx), ctx), v)
    t = q.quantize_tensor(np.arange(8, dtype=np.float32) + 1, q.QuantType.Q8_0, ctx)  # quantize.rs:294-303
    assert t.quant_type == q.QuantType.Q8_0 and t.shape == [8] and t.num_blocks() == 1
    a = q.quantize_tensor(np.arange(256, dtype=np.float32), q.QuantType.Q8_0, ctx)  # quantize.rs:324-335
    b = q.quantize_tensor(np.arange(256, dtype=np.float32), q.QuantType.Q4_0, ctx)
    assert a.compression_ratio() > 2.0 and b.compression_ratio() > a.compression_ratio()


def test_dequantize_block_on_device(ctx):
    img = bytes([0x00, 0x3C] + [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE] * 2)  # types.rs:366-378
    y = q.dequantize_block(np.frombuffer(img, np.uint8), q.QuantType.Q4_0, ctx)
    assert y.tolist() == [float(v) for v in list(range(-8, 8)) * 2]


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("shape", [(1, 256), (3, 512), (7, 2048), (5, 4096 + 256), (64, 11008)])
def test_weight_upload_download_is_identity(ctx, qtype, shape):
    n, k = shape
    if qtype in SUPER and k % 256:
        pytest.skip("k must be a multiple of 256 for the superblock types")
    w = gen_weight(np.random.default_rng(n * 1000 + k), n, k, outlier_p=0.01)
    packed = o.quantize(qtype, w)
    dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], qtype, packed), ctx)
    back = dw.download()
    dw.free()
    assert np.array_equal(back.data, packed)


@pytest.mark.parametrize("qtype", BLOCK)
def test_weight_quantize_on_device_matches_oracle(ctx, qtype):
    n, k = 16, 4096
    w = gen_weight(np.random.default_rng(5), n, k, outlier_p=0.01)
    dw = q.DeviceWeight.quantize(w, qtype, ctx)
    got = dw.download().data
    dw.free()
    assert np.array_equal(got, o.quantize(qtype, w))


def test_error_paths(ctx):
    with pytest.raises(q.DataLengthMismatch):
        q.QuantizedTensor([64], q.QuantType.Q8_0, np.zeros(10, np.uint8))
    qt = q.QuantizedTensor([2, 100], q.QuantType.F32, np.zeros(800, np.uint8))
    qt.quant_type = q.QuantType.Q4_0
    qt.data = np.zeros(126, np.uint8)
    with pytest.raises(q.InvalidBlockSize):  # k = 100 is not a multiple of 32
        q.DeviceWeight.upload(qt, ctx)
    with pytest.raises(q.ShapeMismatch):
        q.DeviceWeight.upload(q.QuantizedTensor([64], q.QuantType.Q8_0, np.zeros(68, np.uint8)), ctx)
    st = ctx.lib.axq_quantize(ctx.handle, 42, None, 32, None, 0)
    assert st == -2 and b"Invalid quantization type" in ctx.lib.axq_last_error(ctx.handle)
