"""Beam search bookkeeping (generation.rs:277-400): the reference's unit test, steps worked by hand, and
(GPU) the driver over the decode model against the same bookkeeping fed by the CPU decode oracle."""
import numpy as np
import pytest

from axonml_amd.generation import Beam, BeamSearch, beam_search_generate


def test_reference_unit_test_init():
    bs = BeamSearch(3, 1.0, False, [0])
    beams = bs.init_beams(np.array([[1, 2, 3]], dtype=np.uint32))
    assert len(beams) == 1 and beams[0].tokens == [1, 2, 3] and beams[0].score == 0.0 and not beams[0].finished


def test_expand_by_hand():
    bs = BeamSearch(2, 1.0, False, [3])
    beams = bs.init_beams([7])
    # one beam, logits over five tokens: the 2 * 2 largest are tokens 1 (5.0), 3 (4.0), 2 (3.0), 4 (2.0)
    beams = bs.expand_beams(beams, [np.array([1.0, 5.0, 3.0, 4.0, 2.0], np.float32)])
    # normalised by length 2: 2.5 and 2.0; token 3 ends its beam
    assert [(b.tokens, float(b.score), b.finished) for b in beams] == [([7, 1], 5.0, False), ([7, 3], 4.0, True)]
    # second step: the finished beam is carried as it is (score 4 / 2 = 2.0) and needs no logits; the live one grows to
    # length 3: token 0 (2.0) -> 7 / 3 = 2.33, token 4 (0.5) -> 5.5 / 3 = 1.83, ...
    beams = bs.expand_beams(beams, [np.array([2.0, -1.0, 0.0, -2.0, 0.5], np.float32), None])
    assert [(b.tokens, float(b.score), b.finished) for b in beams] == [([7, 1, 0], 7.0, False), ([7, 3], 4.0, True)]
    assert bs.best_sequence(beams) == [7, 3]  # only finished beams compete when there is one
    assert not bs.should_stop(beams)          # early_stopping is off


def test_ties_and_length_penalty():
    bs = BeamSearch(2, 1.0, False, [])
    # equal logits: the stable sort keeps lower ids first, among beams and among candidates
    beams = bs.expand_beams(bs.init_beams([0]), [np.array([1.0, 1.0, 1.0, 1.0, 1.0, 1.0], np.float32)])
    assert [b.tokens for b in beams] == [[0, 0], [0, 1]]
    beams = bs.expand_beams(beams, [np.array([0.0, 2.0, 2.0], np.float32), np.array([2.0, 0.0, 2.0], np.float32)])
    assert [b.tokens for b in beams] == [[0, 0, 1], [0, 0, 2]]  # four candidates at 3.0 / 3: the first beam's come first
    # length penalty 0: raw scores compete, a long beam with a larger sum beats a short finished one; penalty 2 turns it round
    long_, short = Beam([1, 2, 3, 4], np.float32(6.0), True), Beam([1, 2], np.float32(4.0), True)
    assert BeamSearch(2, 0.0, False, []).best_sequence([short, long_]) == [1, 2, 3, 4]
    assert BeamSearch(2, 2.0, False, []).best_sequence([short, long_]) == [1, 2]  # 4 / 4 against 6 / 16
    assert float(long_.normalized_score(0.5)) == 3.0
    # equal normalised scores: the last of them (Iterator::max_by)
    a, b = Beam([1, 2], np.float32(2.0), True), Beam([3, 4], np.float32(2.0), True)
    assert BeamSearch(2, 1.0, False, []).best_sequence([a, b]) == [3, 4]
    # nothing finished: the first beam; no beams: nothing
    assert BeamSearch(2, 1.0, False, []).best_sequence([Beam([5]), Beam([6])]) == [5]
    assert BeamSearch(2, 1.0, False, []).best_sequence([]) is None


def test_early_stopping_and_errors():
    bs = BeamSearch(1, 1.0, True, [2])
    beams = bs.expand_beams(bs.init_beams([0]), [np.array([0.0, 1.0, 3.0], np.float32)])
    assert beams[0].finished and bs.should_stop(beams)
    assert not bs.should_stop([Beam([0]), beams[0]])
    with pytest.raises(ValueError):
        bs.expand_beams(bs.init_beams([0]), [np.array([0.0, np.nan], np.float32)])
    # negative infinity is an ordinary value
    beams = BeamSearch(2, 1.0, False, []).expand_beams([Beam([0])], [np.array([-np.inf, 0.0, -np.inf], np.float32)])
    assert [b.tokens for b in beams] == [[0, 1], [0, 0]]


class _OracleSequenceModel:
    """forward_tokens / truncate / reset on the CPU decode oracle (which overwrites cache rows by position)."""

    def __init__(self, cpu):
        self.cpu, self.n = cpu, 0

    def seq_len(self):
        return self.n

    def reset(self):
        self.n = 0

    def truncate(self, n):
        assert n <= self.n
        self.n = n

    def forward_tokens(self, tokens):
        for t in tokens:
            nxt, logits = self.cpu.forward(int(t), self.n)
            self.n += 1
        return nxt, logits


@pytest.mark.gpu
@pytest.mark.parametrize("batched", [False, True])
@pytest.mark.parametrize("num_beams,length_penalty", [(1, 1.0), (3, 1.0), (4, 0.0), (8, 1.5), (2, 1.0), (11, 1.0)])
def test_driver_against_the_oracle(ctx, num_beams, length_penalty, batched):
    """batched: every beam in a sequence slot of the model, one batched step per search step, forks copy their slot;
    otherwise one sequence, rewound and re-fed per beam.  Both against the same bookkeeping over the CPU oracle."""
    if batched and num_beams == 1:
        pytest.skip("one beam needs no slots")
    from tests.decode_common import load_gpu, load_oracle, random_weights, tiny_config

    c = tiny_config(num_layers=2, max_seq_len=64)
    w = random_weights(c, 90 + num_beams)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    prompt = np.random.default_rng(num_beams).integers(0, c["vocab_size"], size=11)
    eos = [5, 17]
    want_seq, want_beams = beam_search_generate(_OracleSequenceModel(cpu), prompt, BeamSearch(num_beams, length_penalty, True, eos), 12)
    got_seq, got_beams = beam_search_generate(gpu, prompt, BeamSearch(num_beams, length_penalty, True, eos), 12, batched=batched)
    assert got_seq == want_seq
    assert [b.tokens for b in got_beams] == [b.tokens for b in want_beams]
    for g, r in zip(got_beams, want_beams):
        assert abs(float(g.score) - float(r.score)) <= 1e-3 * max(1.0, abs(float(r.score))) * len(r.tokens)
    if num_beams == 1:  # one beam is the greedy walk
        gpu.reset()
        greedy, _, _ = gpu.generate(prompt, 12)
        n = len(got_seq) - len(prompt)
        assert got_seq[len(prompt):] == greedy.tolist()[:n]
    gpu.close()
    cpu.close()
