"""Committed vectors (tests/golden/blocks.npz, written by tests/golden/make_fixtures.py from the CPU oracle):
the oracle must still reproduce them, and the GPU path must match them without the oracle in the loop."""
import os

import numpy as np
import pytest

import oracle as o

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "blocks.npz"), allow_pickle=False)
TYPES = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.F16, o.F32, o.Q4_K, o.Q6_K, o.Q5_K]


@pytest.mark.parametrize("t", TYPES)
def test_oracle_reproduces_committed_vectors(t):
    name = o.TYPE_NAMES[t]
    block = 256 if t in (o.Q4_K, o.Q6_K, o.Q5_K) else 32
    for row, packed, deq in zip(GOLD[f"{name}.kat_in"], GOLD[f"{name}.kat_packed"], GOLD[f"{name}.kat_deq"]):
        assert np.array_equal(o.quantize(t, row), packed)
        assert np.array_equal(o.dequantize(t, packed, block), deq)
    w = GOLD["w"]
    assert np.array_equal(o.quantize(t, w), GOLD[f"{name}.packed"])
    assert np.array_equal(o.dequantize(t, GOLD[f"{name}.packed"], w.size).reshape(w.shape), GOLD[f"{name}.deq"])


def test_zero_block_bytes_are_the_hand_computed_ones():
    # zero block: scale 1.0 = 0x3C00 little-endian, Q8_0 codes 0, Q4_0 nibbles 8|8<<4 (quantize.rs:100,139)
    assert GOLD["Q8_0.kat_packed"][0].tolist() == [0x00, 0x3C] + [0] * 32
    assert GOLD["Q4_0.kat_packed"][0].tolist() == [0x00, 0x3C] + [0x88] * 16
    assert GOLD["Q4_1.kat_packed"][0].tolist() == [0x00, 0x3C, 0x00, 0x00] + [0] * 16


@pytest.mark.gpu
@pytest.mark.parametrize("t", TYPES)
def test_gpu_matches_committed_vectors(ctx, t):
    from axonml_amd import quant as q
    from tests.util import MATMUL_RTOL, STRICT_FLOOR, max_rel_err

    name = o.TYPE_NAMES[t]
    w, x = GOLD["w"], GOLD["x"]
    qt = q.quantize_tensor(w, q.QuantType(t), ctx)
    assert np.array_equal(qt.data, GOLD[f"{name}.packed"])
    assert np.array_equal(q.dequantize_tensor(qt, ctx), GOLD[f"{name}.deq"])
    for row, packed in zip(GOLD[f"{name}.kat_in"], GOLD[f"{name}.kat_packed"]):
        assert np.array_equal(q.quantize_tensor(row, q.QuantType(t), ctx).data, packed)
    y = q.quantized_matmul(x, qt, None, ctx)
    assert max_rel_err(y, GOLD[f"{name}.y64"], STRICT_FLOOR) <= MATMUL_RTOL
