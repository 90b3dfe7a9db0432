"""GPU parity at the benchmark configurations' own weight sizes and at depth.

1. The device quantisers against the oracle's (quantize.rs:82-205) on the very weights the configurations
   name -- 4096 x 4096 (Q8_0), 11008 x 4096 (Q4_0, Q4_1), 14336 x 4096 (Q4_K, Q5_1): every packed byte equal.
2. Config 4 at depth: LLaMA::forward_with_cache loops over all layers (llama.rs:731-762; 32 in
   mistral.rs:56-70).  Eight layers of the real shape against the CPU decode oracle (its f32 weights of
   eight layers take 7.5 GB of host memory; 32 would take 28 GB and minutes per token): a 512-token prompt,
   then 16 greedy one-token steps, ids and logits.
3. The 32-layer model itself (random init on the device, no oracle at that size) through properties that do
   not depend on the size: two runs give the same ids, graph replay and plain launches give the same ids, the
   prompt path and the one-token path agree on the next id, logits are finite.
"""
import ctypes as C
import subprocess
import sys

import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from axonml_amd._lib import MEM_DEVICE
from tests.decode_common import LIN_SHAPES, load_gpu, load_oracle, tiny_config
from tests.util import DECODE_FLOOR, DECODE_RTOL, max_rel_err

pytestmark = pytest.mark.gpu


def device_normal(ctx, n, std, outlier_p, seed):
    """n floats ~N(0, std) with a fraction outlier_p at +-0.5, drawn on the device (fast), as a host array."""
    d = ctx.malloc(n * 4)
    ctx.check(ctx.lib.axq_fill_normal_f32(ctx.handle, d, n, 0.0, std, outlier_p, 0.5, seed))
    out = ctx.to_host(d, (n,), np.float32)
    ctx.free(d)
    return out


@pytest.mark.parametrize("qtype,n,k,outliers", [(o.Q8_0, 4096, 4096, 0.0), (o.Q4_0, 11008, 4096, 0.0), (o.Q4_1, 11008, 4096, 0.0),
                                                (o.Q4_K, 14336, 4096, 0.01), (o.Q5_1, 14336, 4096, 0.0), (o.Q6_K, 4096, 14336, 0.01), (o.Q5_K, 4096, 4096, 0.01)])
def test_device_quantiser_is_bit_exact_at_the_configs_own_sizes(ctx, qtype, n, k, outliers):
    w = device_normal(ctx, n * k, 0.02, outliers, 900 + qtype)
    assert np.isfinite(w).all() and 0.015 < w.std() < (0.06 if outliers else 0.025)
    want = o.quantize(qtype, w)
    # quantize_tensor: flat f32 -> packed image
    got = q.quantize_tensor(w, qtype, ctx).data
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"{o.TYPE_NAMES[qtype]} {n}x{k}: {bad.size} packed bytes differ, first at {bad[0]}"
    # the weight route the benchmark takes: f32 on the device -> planar weight -> image back
    dw = q.DeviceWeight.quantize(w.reshape(n, k), qtype, ctx)
    back = dw.download().data
    dw.free()
    assert np.array_equal(back, want)


DEPTH = 8


@pytest.fixture(scope="module")
def eight_layers(ctx):
    c = tiny_config(vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_layers=DEPTH, num_heads=32, num_kv_heads=8,
                    head_dim=128, max_seq_len=544)
    rng = np.random.default_rng(8800)
    seed = [8800]

    def lin(n, k):
        seed[0] += 1
        return o.quantize(o.Q4_K, device_normal(ctx, n * k, 0.02, 0.0, seed[0]))

    w = {"emb": (rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.7).astype(np.float16).view(np.uint16),
         "final_norm": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32), "layers": [], "qtype": o.Q4_K}
    for _ in range(DEPTH):
        L = {"norm0": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32),
             "norm1": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32)}
        for name, (n, k) in LIN_SHAPES(c).items():
            L[name] = lin(n, k)
        w["layers"].append(L)
    w["head"] = lin(c["vocab_size"], c["hidden_size"])
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    del w
    yield c, cpu, gpu
    gpu.close()
    cpu.close()


def test_config4_eight_layers_prompt_512_then_16_steps(eight_layers):
    c, cpu, gpu = eight_layers
    prompt = np.random.default_rng(81).integers(0, c["vocab_size"], size=512)
    for pos, t in enumerate(prompt):
        c_next, c_logits = cpu.forward(int(t), pos, want_logits=(pos == 511))
    g_next, g_logits = gpu.forward_tokens(prompt)
    worst = max_rel_err(g_logits, c_logits, DECODE_FLOOR)
    assert worst <= DECODE_RTOL, f"prompt logits at depth {DEPTH}: {worst:.2e}"
    assert g_next == c_next
    tok = c_next
    for pos in range(512, 512 + 16):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        err = max_rel_err(g_logits, c_logits, DECODE_FLOOR)
        worst = max(worst, err)
        assert err <= DECODE_RTOL, (pos, err)
        assert g_next == c_next, pos
        tok = c_next
    print(f"depth {DEPTH}: worst logit error {worst:.2e} of the logit range")


def test_config4_eight_layers_generate_as_the_benchmark_calls_it(eight_layers):
    c, cpu, gpu = eight_layers
    prompt = np.random.default_rng(82).integers(0, c["vocab_size"], size=512)
    gpu.reset()
    got, _, _ = gpu.generate(prompt, 12)
    for pos, t in enumerate(prompt):
        nxt, _ = cpu.forward(int(t), pos, want_logits=False)
    want = []
    for i in range(12):
        want.append(nxt)
        if i + 1 < 12:
            nxt, _ = cpu.forward(nxt, 512 + i, want_logits=False)
    assert got.tolist() == want


# ---- the 32-layer model through size-independent properties

_PLAIN_LAUNCH_SCRIPT = r"""
import sys
import numpy as np
sys.path.insert(0, {root!r})
from axonml_amd import quant as q
from axonml_amd.decode import QuantizedLlama, mistral_7b_config
m = QuantizedLlama(q.default_context(), **mistral_7b_config(160))
m.random_init(q.QuantType.Q4_K, 0.02, 1)
prompt = np.random.default_rng(3).integers(0, 32000, size=96, dtype=np.int32)
ids, _, _ = m.generate(prompt, 24)
print("IDS", " ".join(str(int(t)) for t in ids))
"""


def test_config4_all_32_layers_properties(ctx):
    import os

    from axonml_amd.decode import QuantizedLlama, mistral_7b_config

    m = QuantizedLlama(ctx, **mistral_7b_config(160))
    m.random_init(q.QuantType.Q4_K, 0.02, 1)
    prompt = np.random.default_rng(3).integers(0, 32000, size=96, dtype=np.int32)
    ids, _, _ = m.generate(prompt, 24)
    assert ids.min() >= 0 and ids.max() < 32000
    m.reset()
    again, _, _ = m.generate(prompt, 24)
    assert again.tolist() == ids.tolist()  # graph replays repeat
    # the prompt path (all 96 rows at once through the GEMM) and 96 one-token steps agree on the next id and the logits
    m.reset()
    n_all, l_all = m.forward_tokens(prompt)
    assert np.isfinite(l_all).all() and n_all == ids[0]
    m.reset()
    for t in prompt:
        n_one, l_one = m.forward(int(t))
    assert np.isfinite(l_one).all()
    assert n_one == n_all
    assert max_rel_err(l_all, l_one, DECODE_FLOOR) <= DECODE_RTOL
    # ... and the greedy walk by hand, one forward() per token, gives generate()'s ids
    walk, tok = [], n_one
    for _ in range(24):
        walk.append(tok)
        tok, _ = m.forward(tok, want_logits=False)
    assert walk == ids.tolist()
    m.close()
    # plain launches instead of the captured graph (the knob is read when the library first decodes: a process of its own)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, AXQ_DECODE_GRAPH="0")
    out = subprocess.run([sys.executable, "-c", _PLAIN_LAUNCH_SCRIPT.format(root=root)], env=env, capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    line = [ln for ln in out.stdout.splitlines() if ln.startswith("IDS ")][0]
    assert [int(t) for t in line.split()[1:]] == ids.tolist()
