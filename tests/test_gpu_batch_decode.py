"""GPU parity: several sequences side by side (batched steps, one pass over the weights for all of them)
against the CPU decode oracle walking every sequence on its own.  Bar as for the one-sequence step: greedy
token ids identical, logits within 1e-3 of the logit range."""
import numpy as np
import pytest

import oracle as o
from tests.decode_common import load_gpu, load_oracle, random_weights, tiny_config
from tests.util import DECODE_FLOOR, DECODE_RTOL, max_rel_err

pytestmark = pytest.mark.gpu


def _oracle_walk(cpu, prompt, n_new):
    """Greedy ids and the logits of every step for one prompt (the oracle overwrites cache rows by position)."""
    ids, logits = [], []
    for pos, t in enumerate(prompt):
        nxt, lg = cpu.forward(int(t), pos)
    for i in range(n_new):
        ids.append(nxt)
        logits.append(lg)
        if i + 1 < n_new:
            nxt, lg = cpu.forward(nxt, len(prompt) + i)
    return ids, logits


@pytest.mark.parametrize("n_seq,qtype,over", [(2, o.Q4_K, {}), (8, o.Q4_K, {}), (5, o.Q4_0, dict(num_layers=3)), (3, o.Q8_0, {}),
                                              (4, o.Q5_1, {}),  # outside the small-batch GEMV: rows go one by one
                                              (8, o.Q4_K, dict(num_heads=8, num_kv_heads=2, head_dim=32)),
                                              (3, o.Q4_1, dict(num_heads=2, num_kv_heads=1, head_dim=128)),
                                              (4, o.Q4_K, dict(sliding_window=6)), (1, o.Q4_K, {}),
                                              # more than eight: the linears of a step are GEMMs on f32 rows
                                              (9, o.Q4_K, {}), (24, o.Q4_0, dict(num_heads=8, num_kv_heads=2, head_dim=32)), (44, o.Q5_1, {})])
def test_generate_batch_matches_the_oracle_sequence_by_sequence(ctx, n_seq, qtype, over):
    c = tiny_config(max_seq_len=96, **over)
    w = random_weights(c, 200 + n_seq + qtype, qtype=qtype)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    gpu.set_batch(n_seq)
    rng = np.random.default_rng(n_seq)
    lengths = [[1, 2, 9, 40, 17, 3, 64, 10][i % 8] + i // 8 for i in range(n_seq)]  # ragged: one token, GEMV rows, GEMM rows
    prompts = [rng.integers(0, c["vocab_size"], size=n) for n in lengths]
    n_new = 14
    got, pre_ms, dec_ms = gpu.generate_batch(prompts, n_new)
    assert got.shape == (n_seq, n_new) and pre_ms >= 0 and dec_ms > 0
    for s, p in enumerate(prompts):
        want, _ = _oracle_walk(cpu, p, n_new)
        assert got[s].tolist() == want, s
        assert gpu.seq_len_of(s) == len(p) + n_new - 1
    again, _, _ = gpu.generate_batch(prompts, n_new)  # starts afresh; graph replays are deterministic
    assert np.array_equal(again, got)
    if n_seq == 2:  # longer prompts after the step's graph exists: the row buffers grow, and the graph is taken anew
        longer = [rng.integers(0, c["vocab_size"], size=n) for n in (70, 33)]
        got2, _, _ = gpu.generate_batch(longer, 6)
        for s, p in enumerate(longer):
            want, _ = _oracle_walk(cpu, p, 6)
            assert got2[s].tolist() == want, s
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("n_seq", [3, 8, 12])
def test_generate_batch_with_q_k_v_of_different_block_types(ctx, n_seq):
    """A value projection at six bits and a key projection at eight beside four-bit queries (the mix of GGUF files):
    the odd parts are multiplied apart in the batched step too (small-batch GEMV where it covers the type, row by row
    where it does not, GEMM rows beyond eight sequences)."""
    from tests.decode_common import requantize

    c = tiny_config(max_seq_len=96)
    w = requantize(c, random_weights(c, 260 + n_seq), {(0, "v"): o.Q6_K, (1, "k"): o.Q8_0, (1, "v"): o.Q6_K}, 261)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    gpu.set_batch(n_seq)
    rng = np.random.default_rng(n_seq)
    prompts = [rng.integers(0, c["vocab_size"], size=[1, 5, 40, 12][i % 4] + i) for i in range(n_seq)]
    got, _, _ = gpu.generate_batch(prompts, 10)
    for s, p in enumerate(prompts):
        want, _ = _oracle_walk(cpu, p, 10)
        assert got[s].tolist() == want, s
    gpu.close()
    cpu.close()


def test_forward_batch_logits_at_different_positions(ctx):
    c = tiny_config(max_seq_len=64)
    w = random_weights(c, 300)
    gpu = load_gpu(ctx, c, w)
    n_seq = 4
    gpu.set_batch(n_seq)
    cpus = [load_oracle(c, w) for _ in range(n_seq)]
    # bring the sequences to different positions: sequence 0 through the one-sequence calls, which work on it
    rng = np.random.default_rng(1)
    head = rng.integers(0, c["vocab_size"], size=5)
    for pos, t in enumerate(head):
        cpus[0].forward(int(t), pos)
    gpu.forward_tokens(head, want_logits=False)
    assert gpu.seq_len_of(0) == 5 and gpu.seq_len_of(1) == 0
    toks = [3, 7, 11, 13]
    pos = [5, 0, 0, 0]
    for step in range(12):
        g_next, g_logits = gpu.forward_batch(toks)
        for s in range(n_seq):
            c_next, c_logits = cpus[s].forward(int(toks[s]), pos[s])
            assert max_rel_err(g_logits[s], c_logits, DECODE_FLOOR) <= DECODE_RTOL, (step, s)
            assert g_next[s] == c_next, (step, s)
            pos[s] += 1
        toks = g_next.tolist()
    assert [gpu.seq_len_of(s) for s in range(n_seq)] == pos and gpu.seq_len() == pos[0]
    # the one-sequence step goes on from where the batched ones left sequence 0
    c_next, c_logits = cpus[0].forward(int(toks[0]), pos[0])
    g_next1, g_logits1 = gpu.forward(int(toks[0]))
    assert g_next1 == c_next and max_rel_err(g_logits1, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    gpu.reset()
    assert [gpu.seq_len_of(s) for s in range(n_seq)] == [0] * n_seq
    gpu.close()
    for m in cpus:
        m.close()


def test_batched_sampling_follows_each_sequences_own_history(ctx):
    from axonml_amd.generation import GenerationConfig

    c = tiny_config(max_seq_len=64)
    w = random_weights(c, 310)
    gpu, one = load_gpu(ctx, c, w), load_gpu(ctx, c, w)
    gpu.set_batch(3)
    cfg = GenerationConfig(temperature=0.9, top_k=12, top_p=0.95, repetition_penalty=1.3)
    seed = 99
    gpu.set_sampling(cfg, seed)
    rng = np.random.default_rng(2)
    prompts = [rng.integers(0, c["vocab_size"], size=n) for n in (6, 11, 2)]
    got, _, _ = gpu.generate_batch(prompts, 10)
    for s, p in enumerate(prompts):  # sequence s draws from (seed + s * odd constant, position)
        one.reset()
        one.set_sampling(cfg, (seed + 0x9E3779B97F4A7C15 * s) % (1 << 64))
        want, _, _ = one.generate(p, 10)
        assert got[s].tolist() == want.tolist(), s
    gpu.close()
    one.close()


def test_batch_errors(ctx):
    from axonml_amd import quant as q

    c = tiny_config(num_layers=1)
    m = load_gpu(ctx, c, random_weights(c, 320))
    assert m.batch() == 1
    with pytest.raises(q.QuantError):
        m.set_batch(0)
    with pytest.raises(q.QuantError):
        m.set_batch(65)
    m.set_batch(2)
    assert m.batch() == 2
    with pytest.raises(ValueError):
        m.forward_batch([1])
    with pytest.raises(q.QuantError):
        m.forward_batch([1, 10 ** 6])
    with pytest.raises(q.ShapeMismatch):
        m.generate_batch([[1, 2], []], 3)
    with pytest.raises(q.Overflow):
        m.generate_batch([[1, 2], [3] * c["max_seq_len"]], 3)
    with pytest.raises(q.ShapeMismatch):
        m.generate_batch([[1], [2]], 0)
    for _ in range(c["max_seq_len"]):
        m.forward_batch([1, 2], want_logits=False)
    with pytest.raises(q.Overflow):
        m.forward_batch([1, 2])
    m.set_batch(1)  # back to one sequence, afresh
    assert m.seq_len() == 0
    nxt, _ = m.forward(3)
    assert 0 <= nxt < c["vocab_size"]
    m.close()


def test_copy_sequence_forks_a_prefix(ctx):
    c = tiny_config(max_seq_len=64)
    w = random_weights(c, 330)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    gpu.set_batch(3)
    rng = np.random.default_rng(3)
    prefix = rng.integers(0, c["vocab_size"], size=13)
    gpu.forward_tokens(prefix, want_logits=False)  # sequence 0
    gpu.copy_sequence(0, 2)
    assert [gpu.seq_len_of(s) for s in range(3)] == [13, 0, 13]
    # sequences 0 and 2 go on with different tokens, sequence 1 starts from nothing
    conts = [[5, 6, 7, 8], [9, 10, 11, 12], [200, 201, 202, 203]]
    want = []
    for s, cont in enumerate(conts):
        seq = (list(prefix) if s != 1 else []) + cont
        for pos, t in enumerate(seq):
            nxt, lg = cpu.forward(int(t), pos)
        want.append((nxt, lg))
    for i in range(4):
        g_next, g_logits = gpu.forward_batch([conts[s][i] for s in range(3)])
    for s in range(3):
        assert g_next[s] == want[s][0], s
        assert max_rel_err(g_logits[s], want[s][1], DECODE_FLOOR) <= DECODE_RTOL, s
    with pytest.raises(Exception):
        gpu.copy_sequence(0, 3)
    gpu.close()
    cpu.close()


def test_one_layer_at_the_7b_shape(ctx):
    """The real layer shape (hidden 4096, intermediate 14336, 32 query heads over 8 KV heads of 128, Q4_K) with a
    small vocabulary and one layer, so that the CPU oracle finishes in seconds: the one-token step, a prompt
    through the GEMM rows, the small-batch rows, and batched steps of eight sequences, all against the oracle."""
    c = tiny_config(vocab_size=1024, hidden_size=4096, intermediate_size=14336, num_layers=1, num_heads=32, num_kv_heads=8,
                    head_dim=128, max_seq_len=96)
    w = random_weights(c, 400, std=0.02)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, c["vocab_size"], size=50)  # 49 rows through the GEMM, the last by the one-token step
    for pos, t in enumerate(prompt):
        c_next, c_logits = cpu.forward(int(t), pos)
    g_next, g_logits = gpu.forward_tokens(prompt)
    assert g_next == c_next and max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    tok = c_next
    for pos in range(50, 56):  # one-token steps on top of the cache the rows left
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert g_next == c_next and max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        tok = c_next
    gpu.reset()
    g_next, g_logits = gpu.forward_tokens(prompt[:9])  # eight rows through the small-batch GEMV
    for pos, t in enumerate(prompt[:9]):
        c_next, c_logits = cpu.forward(int(t), pos)
    assert g_next == c_next and max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL
    gpu.set_batch(8)
    prompts = [rng.integers(0, c["vocab_size"], size=n) for n in (3, 40, 1, 12, 9, 2, 35, 5)]
    got, _, _ = gpu.generate_batch(prompts, 5)
    for s, p in enumerate(prompts):
        want, _ = _oracle_walk(cpu, p, 5)
        assert got[s].tolist() == want, s
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("fused_max", ["0", "25", "1000"])
def test_batched_steps_in_both_attention_forms(ctx, monkeypatch, fused_max):
    """Short contexts: one attention workgroup per sequence and head; longer ones: the positions split over workgroups
    and merged, for all sequences in one launch.  The switch-over (normally at 240 positions) is moved into the walk."""
    monkeypatch.setenv("AXQ_ATTN_FUSED_MAX", fused_max)
    c = tiny_config(max_seq_len=80)
    w = random_weights(c, 340)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    gpu.set_batch(5)
    rng = np.random.default_rng(8)
    prompts = [rng.integers(0, c["vocab_size"], size=n) for n in (3, 22, 40, 1, 17)]
    got, _, _ = gpu.generate_batch(prompts, 20)
    for s, p in enumerate(prompts):
        want, _ = _oracle_walk(cpu, p, 20)
        assert got[s].tolist() == want, s
    # logits of single batched steps on top of that, sequences at different positions on both sides of the switch
    toks = got[:, -1].tolist()
    pos = [len(p) + 19 for p in prompts]
    cpus = []
    for s, p in enumerate(prompts):
        m = load_oracle(c, w)
        seq = list(p) + got[s, :-1].tolist()
        for i, t in enumerate(seq):
            m.forward(int(t), i)
        cpus.append(m)
    for step in range(3):
        g_next, g_logits = gpu.forward_batch(toks)
        for s in range(5):
            c_next, c_logits = cpus[s].forward(int(toks[s]), pos[s])
            assert max_rel_err(g_logits[s], c_logits, DECODE_FLOOR) <= DECODE_RTOL, (step, s)
            assert g_next[s] == c_next
            pos[s] += 1
        toks = g_next.tolist()
    gpu.close()
    cpu.close()
    for m in cpus:
        m.close()
