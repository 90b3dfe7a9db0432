"""GPU parity: the decode step against the CPU decode oracle on small models.
Bar: greedy token ids identical; logits within 1e-3 of the logit range (max|y - ref| / max|ref|, see
tests/util.py for why the stack is compared normwise); f16 cache contents identical except for isolated
one-ulp roundings."""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from tests.decode_common import LIN_SHAPES, load_gpu, load_oracle, random_weights, requantize, tiny_config
from tests.util import DECODE_FLOOR, DECODE_RTOL, max_rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q4_0, o.Q8_0, o.Q5_1, o.Q6_K, o.Q5_K])
def test_step_by_step_logits_and_tokens(ctx, qtype):
    c = tiny_config()
    w = random_weights(c, 10 + qtype, qtype=qtype)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    tok = 11
    for pos in range(24):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, (pos, o.TYPE_NAMES[qtype])
        assert g_next == c_next, pos
        tok = c_next
    assert gpu.seq_len() == 24
    gpu.close()


@pytest.mark.parametrize("window", [1, 5, 32, 40])
def test_sliding_window_attention(ctx, window):
    # windows inside one 32-position split, ending exactly on a split, and spanning two splits
    c = tiny_config(sliding_window=window, max_seq_len=100)
    w = random_weights(c, 60 + window)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    tok = 2
    for pos in range(90):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.close()


@pytest.mark.parametrize("fused_max", ["0", "20", "1000"])
def test_both_attention_forms_of_the_step(ctx, monkeypatch, fused_max):
    """Short contexts take one attention workgroup per head, longer ones split the positions over workgroups and
    merge; the switch-over (normally at 1024 positions) is moved into the walk here."""
    monkeypatch.setenv("AXQ_ATTN_FUSED_MAX", fused_max)
    c = tiny_config(max_seq_len=64, sliding_window=0)
    w = random_weights(c, 95)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    tok = 4
    for pos in range(40):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.reset()
    prompt = np.random.default_rng(5).integers(0, c["vocab_size"], size=12)
    want = []
    for pos, t in enumerate(prompt):
        nxt, _ = cpu.forward(int(t), pos)
    for i in range(30):
        want.append(nxt)
        nxt, _ = cpu.forward(nxt, len(prompt) + i)
    got, _, _ = gpu.generate(prompt, 30)  # crosses position 20 inside the generation loop
    assert got.tolist() == want
    gpu.close()
    cpu.close()


def test_kv_cache_matches_oracle_up_to_isolated_f16_roundings(ctx):
    c = tiny_config(num_layers=2)
    w = random_weights(c, 50)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    tok, n = 3, 20
    for pos in range(n):  # both sides are fed the oracle's tokens
        gpu.forward(tok, want_logits=False)
        tok, _ = cpu.forward(tok, pos)
    for layer in range(2):
        for which in (0, 1):
            a, b = cpu.kv(layer, which)[:, :n], gpu.kv(layer, which)[:, :n]
            differ = a != b
            assert differ.mean() < 0.1, (layer, which, differ.mean())  # a few per cent once upstream noise reaches 1e-5
            af, bf = a.view(np.float16).astype(np.float64), b.view(np.float16).astype(np.float64)
            # one f16 ulp of the element; values that are small by cancellation (a rotated key is a difference
            # of two products) carry the upstream f32 noise instead, ~1e-5 of the largest element
            ulp = np.maximum(np.abs(af) * 2.0 ** -10, 5e-5 * np.abs(af).max())
            bad = np.argwhere(np.abs(af - bf) > ulp)
            assert bad.size == 0, f"cache element {bad[0]} differs by more than one f16 ulp: {af[tuple(bad[0])]} vs {bf[tuple(bad[0])]}"
    gpu.close()


def test_generate_matches_oracle_greedy_and_is_repeatable(ctx):
    c = tiny_config(num_layers=3, max_seq_len=160)
    w = random_weights(c, 20)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, c["vocab_size"], size=17)
    want, tok = [], None
    for pos, t in enumerate(prompt):
        tok, _ = cpu.forward(int(t), pos)
    for i in range(128):
        want.append(tok)
        if i + 1 < 128:
            tok, _ = cpu.forward(tok, len(prompt) + i)
    got, pre_ms, dec_ms = gpu.generate(prompt, 128)
    assert got.tolist() == want
    assert gpu.seq_len() == len(prompt) + 127 and pre_ms > 0 and dec_ms > 0
    gpu.reset()
    again, _, _ = gpu.generate(prompt, 128)
    assert again.tolist() == want  # graph replays are deterministic and the reset clears the position
    gpu.close()


def test_f32_embedding_table_as_the_reference_keeps_it(ctx):
    """Embedding::lookup copies f32 rows (nn/src/layers/embedding.rs:103-146).  A table whose values do not fit f16 goes in
    as f32 on both sides; it replaces the f16 table after the step graph has been captured, and the f16 one comes back."""
    c = tiny_config(max_seq_len=64)
    w = random_weights(c, 77)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, c["vocab_size"], size=9)

    def walk(n):
        want = []
        for pos, t in enumerate(prompt):
            tok, _ = cpu.forward(int(t), pos)
        for i in range(n):
            want.append(tok)
            tok, _ = cpu.forward(tok, len(prompt) + i)
        return want

    got, _, _ = gpu.generate(prompt, 12)  # captures the step graph over the f16 table
    assert got.tolist() == walk(12)
    table = (rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.7).astype(np.float32)
    assert not np.array_equal(table.astype(np.float16).astype(np.float32), table)
    gpu.set_embedding_f32(table)
    cpu.set_embedding_f32(table)
    gpu.reset()
    got32, _, _ = gpu.generate(prompt, 12)
    want32 = walk(12)
    assert got32.tolist() == want32 and want32 != got.tolist()
    gpu.reset()
    g_next, g_logits = gpu.forward_tokens(prompt)
    for pos, t in enumerate(prompt):
        c_next, c_logits = cpu.forward(int(t), pos)
    assert g_next == c_next and max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    gpu.set_embedding_f16(w["emb"])
    cpu.set_embedding_f16(w["emb"])
    gpu.reset()
    back, _, _ = gpu.generate(prompt, 12)
    assert back.tolist() == got.tolist()
    with pytest.raises(q.ShapeMismatch):
        gpu.set_embedding_f32(table[:-1])
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("over,qtype,n_first,n_prompt", [
    (dict(), o.Q4_K, 0, 2), (dict(), o.Q4_K, 0, 3), (dict(), o.Q4_K, 0, 9), (dict(), o.Q4_0, 0, 10), (dict(), o.Q8_0, 5, 26),
    (dict(num_layers=3), o.Q4_1, 3, 17),
    (dict(), o.Q5_1, 0, 12), (dict(), o.Q5_1, 0, 6),  # a type outside the small-batch GEMV: GEMM from 8 rows, else one by one
    (dict(num_heads=8, num_kv_heads=2, head_dim=32), o.Q4_K, 1, 20),
    (dict(num_heads=2, num_kv_heads=1, head_dim=128), o.Q4_K, 0, 19),
    (dict(num_heads=1, num_kv_heads=1, head_dim=256), o.Q4_K, 2, 11),
    (dict(sliding_window=5), o.Q4_K, 0, 30), (dict(sliding_window=12, max_seq_len=100), o.Q4_K, 7, 60),
    # from 33 tokens on the rows before the last go through the GEMM (f32 activations as two f16 rows each)
    (dict(max_seq_len=100), o.Q4_K, 0, 70), (dict(max_seq_len=100), o.Q4_0, 3, 45), (dict(max_seq_len=100), o.Q5_0, 0, 34),
    (dict(max_seq_len=128, num_heads=8, num_kv_heads=2, head_dim=32), o.Q8_0, 10, 100),
    (dict(max_seq_len=100, num_heads=2, num_kv_heads=1, head_dim=128, num_layers=3), o.Q4_1, 0, 41),
    # many rows: attention on the matrix pipe; several key tiles per wave, every ratio of query to KV heads, windows
    (dict(max_seq_len=320), o.Q4_K, 0, 300), (dict(max_seq_len=320), o.Q4_K, 37, 270),
    (dict(max_seq_len=200, num_heads=8, num_kv_heads=1, head_dim=32), o.Q4_K, 0, 190),
    (dict(max_seq_len=200, num_heads=4, num_kv_heads=4, head_dim=64), o.Q4_0, 5, 150),
    (dict(max_seq_len=200, num_heads=2, num_kv_heads=2, head_dim=128), o.Q8_0, 0, 130),
    (dict(max_seq_len=260, sliding_window=40), o.Q4_K, 0, 250), (dict(max_seq_len=260, sliding_window=33, num_heads=8, num_kv_heads=2, head_dim=32), o.Q4_K, 9, 240),
    (dict(max_seq_len=200, num_heads=3, num_kv_heads=1, head_dim=64, hidden_size=192), o.Q8_0, 0, 120),  # three query heads per KV head: the general kernel
])
def test_prompt_fed_at_once_matches_the_oracle_token_by_token(ctx, over, qtype, n_first, n_prompt):
    _prompt_at_once(ctx, over, qtype, n_first, n_prompt)


@pytest.mark.parametrize("chunk,over,n_first,n_prompt", [("64", dict(max_seq_len=320), 0, 300), ("100", dict(max_seq_len=320, sliding_window=90), 21, 250),
                                                         ("40", dict(max_seq_len=200, num_heads=8, num_kv_heads=2, head_dim=32), 0, 161)])
def test_prompt_in_several_chunks(ctx, monkeypatch, chunk, over, n_first, n_prompt):
    """A prompt longer than one pass takes (normally 2048 rows; the knob is read when the model is made) goes through
    the layers in chunks: the later ones attend to the keys the earlier ones left, the last may be a single row."""
    monkeypatch.setenv("AXQ_PROMPT_CHUNK", chunk)
    _prompt_at_once(ctx, over, o.Q4_K, n_first, n_prompt)


def _prompt_at_once(ctx, over, qtype, n_first, n_prompt):
    """forward_tokens (up to eight prompt tokens per pass over the weights) against the oracle's one-token steps:
    last logits and next token to the decode bar, and the KV cache against the GPU's own one-token path."""
    c = tiny_config(**over)
    w = random_weights(c, 70 + n_prompt, qtype=qtype)
    cpu, gpu, one = load_oracle(c, w), load_gpu(ctx, c, w), load_gpu(ctx, c, w)
    rng = np.random.default_rng(n_prompt)
    toks = rng.integers(0, c["vocab_size"], size=n_first + n_prompt)
    for pos, t in enumerate(toks):
        c_next, c_logits = cpu.forward(int(t), pos)
        one.forward(int(t), want_logits=False)
    for t in toks[:n_first]:
        gpu.forward(int(t), want_logits=False)
    g_next, g_logits = gpu.forward_tokens(toks[n_first:])
    assert gpu.seq_len() == len(toks)
    assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    assert g_next == c_next
    n = len(toks)
    for layer in range(c["num_layers"]):
        for which in (0, 1):
            a, b = one.kv(layer, which)[:, :n], gpu.kv(layer, which)[:, :n]
            af, bf = a.view(np.float16).astype(np.float64), b.view(np.float16).astype(np.float64)
            ulp = np.maximum(np.abs(af) * 2.0 ** -10, 5e-5 * np.abs(af).max())  # as in the cache test above
            # The first layer's cache sees the same inputs on both paths: f32 noise flips an f16 rounding at most.  Every
            # flipped rounding then reaches the layers above as a difference of 1e-4 of the hidden state, and the two
            # paths (GEMV on integer limbs, GEMM on f16 pairs) round differently, so the allowance grows by one unit per
            # layer; the logits at the end are held to the decode bar against the oracle above.
            bad = np.argwhere(np.abs(af - bf) > (1 + layer) * ulp)
            assert bad.size == 0, (layer, which, bad[0])
    # the two paths go on alike: a few more steps, one token at a time
    tok = c_next
    for pos in range(n, min(n + 4, c["max_seq_len"])):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    for m in (gpu, one):
        m.close()


def test_forward_tokens_errors_leave_the_model_usable(ctx):
    from axonml_amd import quant as q

    c = tiny_config(num_layers=1)
    w = random_weights(c, 41)
    cpu, m = load_oracle(c, w), load_gpu(ctx, c, w)
    with pytest.raises(q.ShapeMismatch):
        m.forward_tokens([])
    with pytest.raises(q.QuantError):
        m.forward_tokens([1, 2, 10 ** 6])
    with pytest.raises(q.Overflow):
        m.forward_tokens(np.zeros(c["max_seq_len"] + 1, np.int32))
    assert m.seq_len() == 0
    toks = [4, 5, 6, 7, 8]
    for pos, t in enumerate(toks):
        c_next, c_logits = cpu.forward(t, pos)
    g_next, g_logits = m.forward_tokens(toks)
    assert g_next == c_next and max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    m.close()


def test_gqa_and_head_dim_variants(ctx):
    for over in (dict(num_heads=8, num_kv_heads=2, head_dim=32), dict(num_heads=2, num_kv_heads=1, head_dim=128),
                 dict(num_heads=4, num_kv_heads=4, head_dim=64, hidden_size=512, intermediate_size=768)):
        c = tiny_config(**over)
        w = random_weights(c, 30)
        cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
        tok = 1
        for pos in range(8):
            c_next, c_logits = cpu.forward(tok, pos)
            g_next, g_logits = gpu.forward(tok)
            assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, (over, pos)
            assert g_next == c_next
            tok = c_next
        gpu.close()


def test_error_paths(ctx):
    from axonml_amd import quant as q
    from axonml_amd.decode import QuantizedLlama

    with pytest.raises(q.ShapeMismatch):
        QuantizedLlama(ctx, vocab_size=64, hidden_size=256, intermediate_size=512, num_hidden_layers=1,
                       num_attention_heads=3, num_key_value_heads=2, head_dim=64, max_position_embeddings=16,
                       rms_norm_eps=1e-5, rope_theta=1e4)
    c = tiny_config(num_layers=1)
    m = load_gpu(ctx, c, random_weights(c, 40))
    with pytest.raises(q.ShapeMismatch):  # wrong linear shape
        m.set_linear(0, "q", q.quantize_tensor(np.zeros((64, 256), np.float32), q.QuantType.Q4_K, ctx))
    with pytest.raises(q.InvalidQuantType):  # the fused gate/up weight holds one type (q, k, v may differ: kept apart)
        m.set_linear(0, "gate", q.quantize_tensor(np.zeros((512, 256), np.float32), q.QuantType.Q8_0, ctx))
    with pytest.raises(q.QuantError):
        m.forward(10 ** 6)
    fresh = QuantizedLlama(ctx, vocab_size=64, hidden_size=256, intermediate_size=512, num_hidden_layers=1,
                           num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=16,
                           rms_norm_eps=1e-5, rope_theta=1e4)
    with pytest.raises(q.InvalidData):  # weights not set
        fresh.forward(1)
    with pytest.raises(q.ShapeMismatch):  # a norm weight that is not hidden_size long
        fresh.set_norm(0, 0, np.ones(255, np.float32))
    with pytest.raises(q.ShapeMismatch):  # an embedding table of the wrong size
        fresh.set_embedding_f16(np.zeros(64 * 255, np.uint16))
    with pytest.raises(KeyError):  # a projection name that does not exist must not land on q_proj
        fresh.set_linear(0, "q_proj", q.quantize_tensor(np.zeros((256, 256), np.float32), q.QuantType.Q4_K, ctx))
    for _ in range(c["max_seq_len"]):
        m.forward(1, want_logits=False)
    with pytest.raises(q.Overflow):  # cache full
        m.forward(1)


@pytest.mark.parametrize("over,n_first,n_prompt", [(dict(max_seq_len=400), 0, 390), (dict(max_seq_len=400, sliding_window=70), 11, 300),
                                                    (dict(max_seq_len=300, num_heads=8, num_kv_heads=1, head_dim=32), 3, 257),
                                                    (dict(max_seq_len=300, num_heads=2, num_kv_heads=2, head_dim=128), 0, 33)])
def test_the_two_prompt_attention_kernels_agree(ctx, monkeypatch, over, n_first, n_prompt):
    """The matrix-pipe attention of prompt rows against the per-query kernel on the same model and tokens: last logits,
    hidden state and the KV cache (rows written by layer 2 depend on layer 1's attention output)."""
    c = tiny_config(num_layers=3, **over)
    w = random_weights(c, 99)
    toks = np.random.default_rng(n_prompt).integers(0, c["vocab_size"], size=n_first + n_prompt)
    out = []
    for knob in ("1", "0"):
        monkeypatch.setenv("AXQ_ATTN_MFMA", knob)
        m = load_gpu(ctx, c, w)
        for t in toks[:n_first]:
            m.forward(int(t), want_logits=False)
        nxt, logits = m.forward_tokens(toks[n_first:])
        out.append((nxt, logits, m.hidden(), [m.kv(l, which)[:, :len(toks)].copy() for l in range(3) for which in (0, 1)]))
        m.close()
    (n1, l1, h1, kv1), (n0, l0, h0, kv0) = out
    assert n1 == n0
    assert max_rel_err(l1, l0, DECODE_FLOOR) <= 1e-4   # both are f32-accurate: they agree far inside the decode bar
    assert max_rel_err(h1, h0, 1e-2) <= 2e-3   # an f16 cache element that rounds the other way moves the last layers by about 1e-5
    for a, b in zip(kv1, kv0):
        af, bf = a.view(np.float16).astype(np.float64), b.view(np.float16).astype(np.float64)
        assert np.abs(af - bf).max() <= 2.0 ** -9 * np.abs(af).max()  # isolated one-ulp f16 roundings at most


def test_wide_layers_in_q8_0(ctx):
    """Hidden and feed-forward widths beyond 8192 in Q8_0: gate/up (fused RMSNorm and SwiGLU, K = 9216: nine K slices, an odd
    count) and down (K = 8448: the ninth slice a quarter full) take the split-wave GEMV whose weight waves cover two
    slices each.  One layer, a few positions, against the oracle."""
    c = tiny_config(hidden_size=9216, intermediate_size=8448, num_layers=1, num_heads=8, num_kv_heads=2, head_dim=64, max_seq_len=16)
    w = random_weights(c, 5, qtype=o.Q8_0, std=0.02)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    tok = 7
    for pos in range(5):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.close()
    cpu.close()


def test_a_linear_set_again_in_another_block_type(ctx):
    """o, down and the lm_head have their slots to themselves: setting one again in another type replaces it (and drops
    the recorded step, which holds the old weight's address); the walk then follows the oracle with the new weights."""
    c = tiny_config(max_seq_len=64)
    w = random_weights(c, 81)
    gpu = load_gpu(ctx, c, w)
    tok = 5
    for _ in range(6):
        tok, _ = gpu.forward(tok)
    w2 = requantize(c, w, {(0, "down"): o.Q6_K, (1, "o"): o.Q8_0, (-1, "head"): o.Q6_K}, 82)
    L = w2["layers"]
    shapes = {"down": (c["hidden_size"], c["intermediate_size"]), "o": (c["hidden_size"], c["num_heads"] * c["head_dim"])}
    gpu.set_linear(0, "down", q.QuantizedTensor(list(shapes["down"]), o.Q6_K, L[0]["down"]))
    gpu.set_linear(1, "o", q.QuantizedTensor(list(shapes["o"]), o.Q8_0, L[1]["o"]))
    gpu.set_linear(-1, "q", q.QuantizedTensor([c["vocab_size"], c["hidden_size"]], o.Q6_K, w2["head"]))
    gpu.reset()
    cpu = load_oracle(c, w2)
    tok = 5
    for pos in range(30):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("changes", [{(0, "v"): o.Q6_K}, {(0, "k"): o.Q8_0, (0, "v"): o.Q6_K, (1, "v"): o.Q5_1},
                                     {(1, "q"): o.Q6_K, (0, "down"): o.Q6_K, (1, "o"): o.Q8_0, (-1, "head"): o.Q6_K}])
def test_q_k_v_of_different_block_types(ctx, changes):
    """GGUF files mix types inside a layer (llama.cpp's Q4_K_M keeps some attn_v at six bits): q, k or v of another type
    than the fused weight is multiplied apart, into its rows of qkv.  One-token steps, the prompt path through the GEMM
    and through the small-batch GEMV, and batched steps, all against the oracle with the same weights."""
    c = tiny_config(max_seq_len=96)
    w = requantize(c, random_weights(c, 70), changes, 71)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    prompt = np.random.default_rng(72).integers(0, c["vocab_size"], size=45)
    for pos, t in enumerate(prompt):
        c_next, c_logits = cpu.forward(int(t), pos)
    g_next, g_logits = gpu.forward_tokens(prompt)  # 44 rows through the GEMM, the last as a one-token step
    assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL and g_next == c_next
    tok = c_next
    for pos in range(45, 53):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    few = [int(t) for t in prompt[:6]]  # six more rows at once: the small-batch GEMV where it covers the types
    for i, t in enumerate(few):
        c_next, c_logits = cpu.forward(t, 53 + i)
    g_next, g_logits = gpu.forward_tokens(few)
    assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL and g_next == c_next
    # going back to the fused weight's own type puts the part back into it
    (l, name), _ = next(iter(changes.items()))
    if l >= 0 and name in ("q", "k", "v"):
        n, k = LIN_SHAPES(c)[name]
        w2 = dict(w, types=dict(w["types"]))
        w2["layers"] = [dict(L) for L in w["layers"]]
        w2["layers"][l][name] = o.quantize(w["qtype"], (np.random.default_rng(73).standard_normal((n, k)) * 0.06).astype(np.float32))
        del w2["types"][(l, name)]
        gpu.set_linear(l, name, q.QuantizedTensor([n, k], w["qtype"], w2["layers"][l][name]))
        gpu.reset()
        cpu2 = load_oracle(c, w2)
        tok = 7
        for pos in range(6):
            c_next, c_logits = cpu2.forward(tok, pos)
            g_next, g_logits = gpu.forward(tok)
            assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL and g_next == c_next
            tok = c_next
        cpu2.close()
    gpu.close()
    cpu.close()
