"""Host-side mirror of the reference's generation utilities (crates/axonml-llm/src/generation.rs) over the
device sampler: `GenerationConfig` with its constructors and builders (:11-121) and `TextGenerator`
(:124-277), whose `get_next_token` runs as one device kernel (`axq_sample_token`).  The reference draws its
uniform variate from `rand::thread_rng`; here the caller passes `u`, or a numpy Generator supplies it.
`Beam` and `BeamSearch` (:277-400) are the reference's bookkeeping over per-beam logits; `beam_search_generate`
drives them with the one-sequence decode model by rewinding its cache to the prefix a beam shares with what the
cache holds and feeding the rest of the beam's tokens at once.
"""
import ctypes as C
import dataclasses
from typing import List, Optional

import numpy as np

from . import _lib
from ._lib import MEM_HOST
from .quant import default_context


@dataclasses.dataclass
class GenerationConfig:
    """Field names and defaults of GenerationConfig (generation.rs:11-53)."""
    max_new_tokens: int = 50
    temperature: float = 1.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    repetition_penalty: float = 1.0
    eos_token_ids: List[int] = dataclasses.field(default_factory=list)
    pad_token_id: Optional[int] = None
    do_sample: bool = True
    num_beams: int = 1
    length_penalty: float = 1.0
    early_stopping: bool = False

    @classmethod
    def greedy(cls):  # :56-64
        return cls(do_sample=False, temperature=1.0, top_k=None, top_p=None)

    @classmethod
    def sampling(cls, temperature):  # :67-73
        return cls(do_sample=True, temperature=temperature)

    @classmethod
    def top_k_sampling(cls, k, temperature):  # :76-83
        return cls(do_sample=True, temperature=temperature, top_k=k)

    @classmethod
    def nucleus_sampling(cls, p, temperature):  # :86-93
        return cls(do_sample=True, temperature=temperature, top_p=p)

    def with_max_tokens(self, max_new_tokens):
        return dataclasses.replace(self, max_new_tokens=max_new_tokens)

    def with_eos_token(self, eos_token_id):
        return dataclasses.replace(self, eos_token_ids=self.eos_token_ids + [int(eos_token_id)])

    def with_repetition_penalty(self, penalty):
        return dataclasses.replace(self, repetition_penalty=penalty)

    def to_c(self):
        return _lib.SamplingConfig(float(self.temperature), int(self.top_k or 0), -1.0 if self.top_p is None else float(self.top_p),
                                   float(self.repetition_penalty), 1 if self.do_sample else 0)


class TextGenerator:
    def __init__(self, config, ctx=None, rng=None):
        self.config = config
        self.ctx = ctx or default_context()
        self.rng = rng or np.random.default_rng()

    def get_next_token(self, logits, generated_tokens=(), u=None, return_filtered=False):
        """generation.rs:258-269.  `u` in [0, 1) replaces the reference's thread_rng draw."""
        lg = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
        gen = np.ascontiguousarray(generated_tokens, dtype=np.int32).reshape(-1)
        if u is None:
            u = float(np.float32(self.rng.random(dtype=np.float32)))
        tok = C.c_int32()
        filtered = np.empty_like(lg) if return_filtered else None
        cfg = self.config.to_c()
        self.ctx.check(self.ctx.lib.axq_sample_token(self.ctx.handle, lg.ctypes.data, lg.size, gen.ctypes.data if gen.size else None,
                                                     gen.size, C.byref(cfg), u, C.byref(tok),
                                                     filtered.ctypes.data if return_filtered else None, MEM_HOST))
        return (tok.value, filtered) if return_filtered else tok.value

    def should_stop(self, token):  # :272-274
        return int(token) in self.config.eos_token_ids


@dataclasses.dataclass
class Beam:
    """Beam (generation.rs:277-304).  `score` adds raw logits in f32, as the reference does."""
    tokens: List[int]
    score: np.float32 = np.float32(0.0)
    finished: bool = False

    def normalized_score(self, length_penalty):
        return np.float32(self.score) / np.power(np.float32(len(self.tokens)), np.float32(length_penalty))


class BeamSearch:
    """BeamSearch (generation.rs:306-400)."""

    def __init__(self, num_beams, length_penalty, early_stopping, eos_token_ids):
        self.num_beams, self.length_penalty = int(num_beams), float(length_penalty)
        self.early_stopping, self.eos_token_ids = bool(early_stopping), [int(t) for t in eos_token_ids]

    def init_beams(self, input_ids):
        return [Beam([int(t) for t in np.asarray(input_ids).reshape(-1)])]

    def expand_beams(self, beams, next_token_logits):
        """Each live beam grows by its 2 * num_beams largest logits (equal logits: lower ids first, a stable
        sort), finished beams stay as they are; the num_beams best by normalised score go on (equal
        scores: in candidate order)."""
        candidates = []
        for beam, logits in zip(beams, next_token_logits):
            if beam.finished:
                candidates.append(beam)
                continue
            logits = np.asarray(logits, dtype=np.float32)
            if np.isnan(logits).any():
                raise ValueError("NaN among the logits")  # partial_cmp(..).unwrap() panics
            order = np.argsort(-logits, kind="stable")[: self.num_beams * 2]
            for token in order:
                token = int(token)
                candidates.append(Beam(beam.tokens + [token], np.float32(beam.score + logits[token]), token in self.eos_token_ids))
        keys = np.array([c.normalized_score(self.length_penalty) for c in candidates], dtype=np.float32)
        if np.isnan(keys).any():
            raise ValueError("NaN among the beam scores")
        keep = np.argsort(-keys, kind="stable")[: self.num_beams]
        return [candidates[i] for i in keep]

    def should_stop(self, beams):
        return self.early_stopping and all(b.finished for b in beams)

    def best_sequence(self, beams):
        """Tokens of the best finished beam (of equal scores the last, Iterator::max_by), else of the first beam."""
        best = None
        for b in beams:
            if b.finished and (best is None or b.normalized_score(self.length_penalty) >= best.normalized_score(self.length_penalty)):
                best = b
        if best is None:
            best = beams[0] if beams else None
        return None if best is None else list(best.tokens)


def beam_search_generate(model, input_ids, beam_search, max_new_tokens, batched=None):
    """Beam search over a `QuantizedLlama`: per step every live beam's next-token logits, then
    `expand_beams`, until `max_new_tokens` or `should_stop`.  Returns (best_sequence, beams).

    batched (default: when the model can and there are 2..64 beams): every beam lives in a sequence slot of the
    model and one batched step serves all of them; a beam that forks copies its slot (`copy_sequence`).
    Otherwise the model keeps one sequence, and a beam is brought in by rewinding the cache to the prefix it
    shares with the cached tokens and feeding the rest (`truncate`, `forward_tokens`)."""
    if batched is None:
        batched = hasattr(model, "forward_batch") and 2 <= beam_search.num_beams <= 64
    if batched:
        return _beam_search_batched(model, input_ids, beam_search, max_new_tokens)
    beams = beam_search.init_beams(input_ids)
    cached = []  # tokens whose keys and values the model's cache holds now
    if model.seq_len():
        model.reset()
    for _ in range(max_new_tokens):
        per_beam = []
        for b in beams:
            if b.finished:
                per_beam.append(None)
                continue
            shared = 0
            limit = min(len(cached), len(b.tokens) - 1)  # at least the last token is fed: its logits are wanted
            while shared < limit and cached[shared] == b.tokens[shared]:
                shared += 1
            model.truncate(shared)
            _, logits = model.forward_tokens(b.tokens[shared:])
            cached = list(b.tokens)
            per_beam.append(logits)
        beams = beam_search.expand_beams(beams, per_beam)
        if beam_search.should_stop(beams):
            break
    return beam_search.best_sequence(beams), beams


def _beam_search_batched(model, input_ids, beam_search, max_new_tokens):
    n_slots = beam_search.num_beams
    if model.batch() != n_slots:
        model.set_batch(n_slots)
    else:
        model.reset()
    beams = beam_search.init_beams(input_ids)
    prompt = beams[0].tokens
    if len(prompt) > 1:
        model.forward_tokens(prompt[:-1], want_logits=False)  # sequence 0
    for s in range(1, n_slots):  # all slots march in step, so idle ones never run ahead of the live ones
        model.copy_sequence(0, s)
    slot_of = {0: 0}  # index into `beams` -> slot, live beams only
    for _ in range(max_new_tokens):
        feed = [0] * n_slots
        for i, slot in slot_of.items():
            feed[slot] = beams[i].tokens[-1]
        _, logits = model.forward_batch(feed)
        per_beam = [logits[slot_of[i]] if i in slot_of else None for i in range(len(beams))]
        grown = beam_search.expand_beams(beams, per_beam)
        # a live beam of the new set continues the old live beam whose tokens it extends by one
        by_tokens = {tuple(beams[i].tokens): slot for i, slot in slot_of.items()}
        parents = [None if b.finished else by_tokens[tuple(b.tokens[:-1])] for b in grown]
        first_child, new_slots = {}, {}
        for j, parent in enumerate(parents):
            if parent is not None and parent not in first_child:
                first_child[parent] = j
                new_slots[j] = parent
        free = [s for s in range(n_slots) if s not in first_child]
        for j, parent in enumerate(parents):
            if parent is not None and j not in new_slots:
                new_slots[j] = free.pop()
                model.copy_sequence(parent, new_slots[j])
        beams, slot_of = grown, new_slots
        if beam_search.should_stop(beams) or not slot_of:
            break
    return beam_search.best_sequence(beams), beams
