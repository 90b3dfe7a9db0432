"""Next-token selection (TextGenerator::get_next_token, llm/src/generation.rs:136-269).

CPU: the oracle against the reference's own test vectors and hand-computed cases.  GPU: the device kernel
against the oracle.  Bar: penalty, temperature and top-k bit-exact; top-p and the draw identical whenever the
cumulative probability stays at least 1e-4 away from its threshold (the reference adds its softmax in f32 one
term after the other, the device adds exactly; see axq_sample.hip), which the tests check in float64 before
they compare."""
import numpy as np
import pytest

import oracle as o
from axonml_amd.generation import GenerationConfig, TextGenerator

MARGIN = 1e-4


# ---------------------------------------------------------------------------
# oracle pins (CPU)
# ---------------------------------------------------------------------------
def test_reference_unit_test_vectors():
    # generation.rs:421-467
    _, f = o.get_next_token([1.0, 5.0, 3.0, 4.0, 2.0], top_k=2, do_sample=False)
    assert np.isfinite(f).sum() == 2 and list(np.flatnonzero(np.isfinite(f))) == [1, 3]
    _, f = o.get_next_token([2.0, 4.0, 6.0], temperature=2.0, do_sample=False)
    assert list(f) == [1.0, 2.0, 3.0]
    tok, _ = o.get_next_token([1.0, 5.0, 3.0, 4.0, 2.0], do_sample=False)
    assert tok == 1
    _, f = o.get_next_token([1.0, 2.0, 3.0, 4.0], generated=[1, 3], repetition_penalty=2.0, do_sample=False)
    assert f[1] < 2.0 and f[3] < 4.0 and list(f) == [1.0, 1.0, 3.0, 2.0]


def test_penalty_compounds_per_occurrence_and_multiplies_non_positive_logits():
    # :145-158: one division (or product) per entry of `generated`, repeats included; 0 is "not > 0"
    _, f = o.get_next_token([8.0, -1.0, 0.0, 3.0], generated=[0, 0, 0, 1, 1, 2, 9], repetition_penalty=2.0, do_sample=False)
    assert list(f) == [1.0, -4.0, 0.0, 3.0]


def test_top_k_ties_keep_the_lower_indices():
    # stable descending sort (:166-167): among the three 2.0 the first two survive k = 3
    _, f = o.get_next_token([2.0, 1.0, 2.0, 5.0, 2.0], top_k=3, do_sample=False)
    assert list(np.isfinite(f)) == [True, False, True, True, False]
    _, f = o.get_next_token([1.0, 2.0], top_k=2, do_sample=False)  # k == len: untouched (:163)
    assert list(f) == [1.0, 2.0]


def test_top_p_keeps_the_element_that_crosses():
    # probabilities 0.5, 0.25, 0.125, 0.125 (logits ln of them): p = 0.6 -> cumsum 0.5, 0.75 > 0.6 -> two kept
    lg = np.log(np.array([0.125, 0.5, 0.125, 0.25], dtype=np.float64)).astype(np.float32)
    _, f = o.get_next_token(lg, top_p=0.6, do_sample=False)
    assert list(np.isfinite(f)) == [False, True, False, True]
    _, f = o.get_next_token(lg, top_p=0.8, do_sample=False)  # 0.5, 0.75, 0.875 > 0.8: the first of the tied 0.125 joins
    assert list(np.isfinite(f)) == [True, True, False, True]
    _, f = o.get_next_token(lg, top_p=1.5, do_sample=False)  # never exceeded: everything stays (:197)
    assert np.isfinite(f).all()
    _, f = o.get_next_token(lg, top_p=0.0, do_sample=False)  # the largest alone already exceeds 0
    assert list(np.isfinite(f)) == [False, True, False, False]


def test_draw_boundaries_and_argmax_ties():
    lg = np.log(np.array([0.25, 0.5, 0.25], dtype=np.float64)).astype(np.float32)
    assert [o.get_next_token(lg, u=u)[0] for u in (0.0, 0.2, 0.3, 0.7, 0.8, 0.99)] == [0, 0, 1, 1, 2, 2]
    assert o.get_next_token([3.0, 7.0, 7.0, 1.0], do_sample=False)[0] == 2  # max_by returns the last maximum
    # filtered-out entries have probability zero and are never drawn
    assert o.get_next_token([0.0, 5.0, 0.0, 5.0], top_k=2, u=0.75)[0] == 3


def test_config_constructors_follow_the_reference():
    c = GenerationConfig()
    assert (c.max_new_tokens, c.temperature, c.do_sample, c.num_beams) == (50, 1.0, True, 1)  # :37-52
    assert not GenerationConfig.greedy().do_sample
    assert GenerationConfig.top_k_sampling(2, 0.7).top_k == 2 and GenerationConfig.nucleus_sampling(0.9, 1.0).top_p == 0.9
    c = GenerationConfig.sampling(0.8).with_max_tokens(7).with_eos_token(2).with_repetition_penalty(1.3)
    assert (c.max_new_tokens, c.eos_token_ids, c.repetition_penalty, c.temperature) == (7, [2], 1.3, 0.8)


# ---------------------------------------------------------------------------
# device kernel (GPU)
# ---------------------------------------------------------------------------
def _cdf64(filtered):
    x = filtered.astype(np.float64)
    e = np.exp(x - x[np.isfinite(x)].max())
    e[~np.isfinite(x)] = 0.0
    return np.cumsum(e / e.sum())


def _logits(rng, n, spread=4.0):
    return (rng.standard_normal(n) * spread).astype(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [5, 1000, 32000, 50257])
@pytest.mark.parametrize("top_k", [None, 1, 40, 2000])
def test_penalty_temperature_top_k_bit_exact(ctx, n, top_k):
    rng = np.random.default_rng(n + (top_k or 0))
    lg = _logits(rng, n)
    lg[rng.integers(0, n, size=max(1, n // 50))] = lg[0]  # ties, some of them at the top-k boundary now and then
    gen = rng.integers(0, n, size=300)
    gen[:20] = gen[20]  # an id repeated twenty-one times
    cfg = GenerationConfig(temperature=0.7, top_k=top_k, repetition_penalty=1.3, do_sample=False)
    tok, f = TextGenerator(cfg, ctx).get_next_token(lg, gen, return_filtered=True)
    want_tok, want = o.get_next_token(lg, gen, temperature=0.7, top_k=top_k, repetition_penalty=1.3, do_sample=False)
    assert np.array_equal(f.view(np.uint32), want.view(np.uint32))
    assert tok == want_tok


@pytest.mark.gpu
def test_top_k_tie_at_the_boundary_keeps_lower_indices(ctx):
    lg = np.full(3000, 1.0, np.float32)
    lg[[5, 77]] = 9.0
    cfg = GenerationConfig(top_k=10, do_sample=False)
    tok, f = TextGenerator(cfg, ctx).get_next_token(lg, return_filtered=True)
    assert list(np.flatnonzero(np.isfinite(f))) == [0, 1, 2, 3, 4, 5, 6, 7, 8, 77]
    assert tok == 77  # the last of the two maxima


@pytest.mark.gpu
@pytest.mark.parametrize("n", [7, 4096, 32000])
@pytest.mark.parametrize("top_k", [None, 50])
def test_top_p_keeps_the_oracles_set(ctx, n, top_k):
    rng = np.random.default_rng(3 * n + (top_k or 0))
    lg = _logits(rng, n, spread=3.0)
    checked = 0
    for p in (0.0, 0.3, 0.5, 0.8, 0.9, 0.95, 0.999, 1.0, 2.0):
        _, want = o.get_next_token(lg, temperature=0.9, top_k=top_k, top_p=p, do_sample=False)
        # skip thresholds that the sorted cumulative probability comes too close to
        _, pre = o.get_next_token(lg, temperature=0.9, top_k=top_k, do_sample=False)
        x = pre.astype(np.float64)
        pr = np.exp(x - x[np.isfinite(x)].max())
        pr[~np.isfinite(x)] = 0
        cs = np.cumsum(np.sort(pr / pr.sum())[::-1])
        if np.abs(cs - p).min() < MARGIN:
            continue
        cfg = GenerationConfig(temperature=0.9, top_k=top_k, top_p=p, do_sample=False)
        tok, f = TextGenerator(cfg, ctx).get_next_token(lg, return_filtered=True)
        assert np.array_equal(np.isfinite(f), np.isfinite(want)), p
        assert np.array_equal(f[np.isfinite(f)], want[np.isfinite(want)])
        checked += 1
    assert checked >= 3  # with 32000 candidates the sorted cumulative sums lie dense near the larger thresholds


@pytest.mark.gpu
def test_top_p_ties_join_in_index_order(ctx):
    lg = np.log(np.array([0.125, 0.5, 0.125, 0.25], dtype=np.float64)).astype(np.float32)
    for p, keep in ((0.6, [1, 3]), (0.8, [0, 1, 3]), (1.5, [0, 1, 2, 3]), (0.0, [1])):
        _, f = TextGenerator(GenerationConfig(top_p=p, do_sample=False), ctx).get_next_token(lg, return_filtered=True)
        assert list(np.flatnonzero(np.isfinite(f))) == keep, p


@pytest.mark.gpu
@pytest.mark.parametrize("n,top_k,top_p", [(5, None, None), (32000, None, None), (32000, 40, None), (32000, 40, 0.9),
                                           (50257, None, 0.95), (1000, 1, None)])
def test_draws_match_the_oracle(ctx, n, top_k, top_p):
    rng = np.random.default_rng(n + 7 * (top_k or 0))
    lg = _logits(rng, n, spread=2.5)
    gen = rng.integers(0, n, size=64)
    cfg = GenerationConfig(temperature=0.8, top_k=top_k, top_p=top_p, repetition_penalty=1.1, do_sample=True)
    g = TextGenerator(cfg, ctx)
    _, filtered = o.get_next_token(lg, gen, temperature=0.8, top_k=top_k, top_p=top_p, repetition_penalty=1.1, u=0.5)
    cdf = _cdf64(filtered)
    checked = 0
    for u in list(rng.random(40).astype(np.float32)) + [0.0, 0.999999]:
        u = float(u)
        if np.abs(cdf - u).min() < MARGIN:
            continue
        want, _ = o.get_next_token(lg, gen, temperature=0.8, top_k=top_k, top_p=top_p, repetition_penalty=1.1, u=u)
        assert g.get_next_token(lg, gen, u=u) == want, u
        checked += 1
    assert checked >= 10


@pytest.mark.gpu
def test_argument_checks(ctx):
    from axonml_amd import quant as q

    lg = np.zeros(8, np.float32)
    for bad in (GenerationConfig(temperature=0.0), GenerationConfig(repetition_penalty=-1.0), GenerationConfig(top_k=-3)):
        with pytest.raises(q.QuantError):
            TextGenerator(bad, ctx).get_next_token(lg, u=0.5)
    with pytest.raises(q.QuantError):
        TextGenerator(GenerationConfig(), ctx).get_next_token(lg, u=1.0)
    assert TextGenerator(GenerationConfig().with_eos_token(3), ctx).should_stop(3)


def _uniform_from(seed, counter):
    """The device's draw for (seed, position): splitmix64, top 24 bits."""
    m = (1 << 64) - 1
    z = (seed + 0x9E3779B97F4A7C15 * (counter + 1)) & m
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
    z ^= z >> 31
    return float(np.float32(z >> 40) * np.float32(1.0 / 16777216.0))


@pytest.mark.gpu
@pytest.mark.parametrize("cfg", [GenerationConfig(do_sample=False, repetition_penalty=1.5),
                                 GenerationConfig(temperature=0.9, top_k=20, top_p=0.9, repetition_penalty=1.2)])
def test_model_generates_with_the_sampler(ctx, cfg):
    from tests.decode_common import load_gpu, random_weights, tiny_config

    c = tiny_config(max_seq_len=64)
    gpu = load_gpu(ctx, c, random_weights(c, 91))
    prompt, n_new, seed = [3, 17, 3, 200], 24, 1234
    gpu.set_sampling(cfg, seed)
    got, _, _ = gpu.generate(prompt, n_new)
    again = None
    gpu.reset()
    again, _, _ = gpu.generate(prompt, n_new)
    assert np.array_equal(got, again)  # draws depend on (seed, position) only
    # the same walk by hand: the model's logits, the oracle's selection over every token fed so far
    gpu.reset()
    gpu.set_sampling(None)
    fed, want, tok = [], [], None
    for t in prompt:
        fed.append(t)
        _, logits = gpu.forward(t)
    ambiguous = False
    for i in range(n_new):
        u = _uniform_from(seed, len(fed))
        tok, filtered = o.get_next_token(logits, fed, temperature=cfg.temperature, top_k=cfg.top_k, top_p=cfg.top_p,
                                         repetition_penalty=cfg.repetition_penalty, do_sample=cfg.do_sample, u=u)
        if cfg.do_sample and np.abs(_cdf64(filtered) - u).min() < MARGIN:
            ambiguous = True
            break
        want.append(tok)
        if i + 1 < n_new:
            fed.append(tok)
            _, logits = gpu.forward(tok)
    assert len(want) >= 8 or not ambiguous
    assert list(got[:len(want)]) == want
    # and greedy is what it was before a sampler was set
    gpu.reset()
    plain, _, _ = gpu.generate(prompt, 8)
    gpu.reset()
    gpu.set_sampling(GenerationConfig.greedy(), 0)
    assert np.array_equal(gpu.generate(prompt, 8)[0], plain)
    gpu.close()


@pytest.mark.gpu
@pytest.mark.parametrize("n", [300, 32000])
def test_small_top_k_with_ties_at_the_cut(ctx, n):
    # the short candidate-list path: six equal logits straddle rank k, the lower indices must win; then top-p and draws
    rng = np.random.default_rng(n)
    lg = _logits(rng, n, spread=2.0)
    order = np.argsort(-lg, kind="stable")
    tied = np.sort(order[36:42])
    lg[tied] = lg[order[38]]
    for top_p in (None, 0.7):
        cfg = GenerationConfig(temperature=1.3, top_k=40, top_p=top_p, repetition_penalty=1.2, do_sample=True)
        gen = rng.integers(0, n, size=50)
        _, want = o.get_next_token(lg, gen, temperature=1.3, top_k=40, top_p=top_p, repetition_penalty=1.2, u=0.5)
        g = TextGenerator(cfg, ctx)
        _, f = g.get_next_token(lg, gen, u=0.5, return_filtered=True)
        if top_p is None:
            assert np.array_equal(f.view(np.uint32), want.view(np.uint32))
            assert np.isfinite(f).sum() == 40
        else:
            _, pre = o.get_next_token(lg, gen, temperature=1.3, top_k=40, repetition_penalty=1.2, u=0.5)
            cs = np.cumsum(np.sort(np.diff(np.concatenate([[0.0], _cdf64(pre)])))[::-1])
            if np.abs(cs - top_p).min() >= MARGIN:
                assert np.array_equal(np.isfinite(f), np.isfinite(want))
        cdf = _cdf64(want)
        for u in (0.01, 0.3, 0.62, 0.97):
            if np.abs(cdf - u).min() >= MARGIN:
                assert g.get_next_token(lg, gen, u=u) == o.get_next_token(lg, gen, temperature=1.3, top_k=40, top_p=top_p,
                                                                           repetition_penalty=1.2, u=u)[0], (top_p, u)
