"""GPU parity at the benchmark configurations' own sizes.

Config 4 (7B-shape decode): the real layer shape (hidden 4096, FFN 14336, 32 query heads over 8 KV heads of
128, Q4_K linears), the real vocabulary (32000: lm_head and argmax at full width), a 512-token prompt and
one-token steps at positions 512 and beyond, which is where the benchmark runs -- the split form of the
one-token attention at head size 128 with four query heads per KV head, and the 511-row prompt pass.  Two
layers instead of 32 keep the CPU decode oracle at seconds; every kernel instantiation is the 32-layer
model's.

Config 5 (prefill GEMM): all six (M, N) shapes at K = 4096 for Q4_K, Q5_K and Q5_1.  The GPU computes the whole
[M, N] product; the oracle gets a random subset of the weight rows (output columns) and the matching
columns are compared, which keeps the single-thread reference sgemm at a second per case.
"""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from tests.decode_common import load_gpu, load_oracle, random_weights, tiny_config
from tests.util import DECODE_FLOOR, DECODE_RTOL, MATMUL_RTOL, STRICT_FLOOR, gen_weight, max_rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def seven_b_slice(ctx):
    c = tiny_config(vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_layers=2, num_heads=32, num_kv_heads=8,
                    head_dim=128, max_seq_len=640)
    w = random_weights(c, 4400, std=0.02)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    yield c, cpu, gpu
    gpu.close()
    cpu.close()


def test_config4_prompt_512_then_steps_beyond(seven_b_slice):
    c, cpu, gpu = seven_b_slice
    rng = np.random.default_rng(44)
    prompt = rng.integers(0, c["vocab_size"], size=512)
    gpu.reset()
    for pos, t in enumerate(prompt):
        c_next, c_logits = cpu.forward(int(t), pos)
    g_next, g_logits = gpu.forward_tokens(prompt)
    assert g_next == c_next
    assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    tok = c_next
    for pos in range(512, 512 + 20):  # greedy one-token steps: split attention <128, 4>, lm_head 32000, argmax
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    assert gpu.seq_len() == 532


def test_config4_generate_matches_the_oracle_walk(seven_b_slice):
    """axq_model_generate as the benchmark calls it (graph replay, ids fed back on the device)."""
    c, cpu, gpu = seven_b_slice
    rng = np.random.default_rng(45)
    prompt = rng.integers(0, c["vocab_size"], size=512)
    gpu.reset()
    got, _, _ = gpu.generate(prompt, 24)
    want = []
    for pos, t in enumerate(prompt):
        nxt, _ = cpu.forward(int(t), pos)
    for i in range(24):
        want.append(nxt)
        if i + 1 < 24:
            nxt, _ = cpu.forward(nxt, 512 + i)
    assert got.tolist() == want


def test_config4_eight_sequences_beyond_240_positions(seven_b_slice):
    """Batched steps in the split attention form at head size 128: eight sequences whose contexts lie beyond the
    switch-over, at different positions."""
    c, cpu, gpu = seven_b_slice
    rng = np.random.default_rng(46)
    lens = (250, 300, 262, 277, 251, 290, 245, 256)
    prompts = [rng.integers(0, c["vocab_size"], size=n) for n in lens]
    gpu.set_batch(8)
    got, _, _ = gpu.generate_batch(prompts, 6)
    toks = got[:, -1].tolist()
    g_next, g_logits = gpu.forward_batch(toks)
    for s, p in enumerate(prompts):
        for pos, t in enumerate(p):
            nxt, _ = cpu.forward(int(t), pos)
        want = []
        for i in range(6):
            want.append(nxt)
            nxt, logits = cpu.forward(nxt, len(p) + i)
        assert got[s].tolist() == want, s
        assert max_rel_err(g_logits[s], logits, DECODE_FLOOR) <= DECODE_RTOL, s
        assert g_next[s] == nxt, s
    gpu.set_batch(1)


@pytest.fixture(scope="module")
def prefill_weights():
    """One weight per (type, N) for the whole module: quantised once on the host by the oracle."""
    cache = {}

    def get(qtype, n):
        if (qtype, n) not in cache:
            rng = np.random.default_rng(1000 + n + qtype)
            cache[(qtype, n)] = o.quantize(qtype, gen_weight(rng, n, 4096))
        return cache[(qtype, n)]

    return get


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q5_1])
@pytest.mark.parametrize("n", [4096, 14336])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_config5_prefill_gemm_full_shapes(ctx, prefill_weights, qtype, m, n):
    k = 4096
    wq = prefill_weights(qtype, n)
    rng = np.random.default_rng(m * 3 + n + qtype)
    xb = q.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    x = q.bf16_bits_to_f32(xb)
    got = q.quantized_matmul_bf16(xb, q.QuantizedTensor([n, k], qtype, wq), ctx)
    assert got.shape == (m, n)
    assert np.isfinite(got).all()
    # 96 random output columns, the tile edges among them
    cols = np.unique(np.concatenate([rng.choice(n, size=90, replace=False), [0, 127, 128, n - 129, n - 128, n - 1]]))
    bpr = o.packed_bytes(qtype, k)  # bytes of one weight row
    sub = np.ascontiguousarray(wq.reshape(n, bpr)[cols]).reshape(-1)
    want = o.matmul_ref(qtype, sub, x, len(cols), k)
    err = max_rel_err(got[:, cols], want)
    assert err <= MATMUL_RTOL, f"{o.TYPE_NAMES[qtype]} M={m} N={n}: max rel err {err:.3e}"
    exact = o.matmul_f64(o.dequantize(qtype, sub, len(cols) * k).reshape(len(cols), k), x)
    assert max_rel_err(got[:, cols], exact, STRICT_FLOOR) <= MATMUL_RTOL


def test_quantize_model_keeps_names_and_order_and_stops_at_the_first_error(ctx):
    """quantize_model (quantize.rs:64-75): every tensor through quantize_tensor, names and order kept; the first
    failing tensor fails the whole call."""
    rng = np.random.default_rng(8)
    tensors = [(f"layers.{i}.w", rng.standard_normal(shape).astype(np.float32)) for i, shape in
               enumerate([(4, 64), (96,), (3, 5, 32), (1, 40)])]
    out = q.quantize_model(tensors, q.QuantType.Q4_1, ctx)
    assert [n for n, _ in out] == [n for n, _ in tensors]
    for (name, t), (_, qt) in zip(tensors, out):
        assert qt.shape == list(t.shape) and qt.quant_type == q.QuantType.Q4_1
        assert np.array_equal(qt.data, o.quantize(o.Q4_1, t)), name
    assert q.quantize_model([], q.QuantType.Q8_0, ctx) == []
    bad = tensors[:2] + [("broken", np.array(["not", "numbers"]))] + tensors[2:]
    with pytest.raises(Exception):
        q.quantize_model(bad, q.QuantType.Q8_0, ctx)
    with pytest.raises(q.InvalidQuantType):
        q.quantize_model(tensors, 99, ctx)


def test_the_grid_barrier_probe_completes(ctx):
    """bench.py --grid-barrier's entry point: every round completes within its bounded wait, with one counter and with two
    levels, and reports times of a plausible size (microseconds, not milliseconds)."""
    import ctypes as C
    out = (C.c_float * 3)()
    for levels, publish in ((1, 0), (2, 1024)):
        ctx.check(ctx.lib.axq_bench_grid_barrier(ctx.handle, levels, publish, 16, out))
        assert 0.0 < out[0] <= out[1] < 1000.0 and 0.0 <= out[2] < 1000.0
    assert ctx.lib.axq_bench_grid_barrier(ctx.handle, 3, 0, 16, out) != 0  # no such form
