"""Host-side mirror of the reference's generation utilities (crates/axonml-llm/src/generation.rs) over the
device sampler: `GenerationConfig` with its constructors and builders (:11-121) and `TextGenerator`
(:124-277), whose `get_next_token` runs as one device kernel (`axq_sample_token`).  The reference draws its
uniform variate from `rand::thread_rng`; here the caller passes `u`, or a numpy Generator supplies it.
Beam search (:279-400) needs several sequences in flight and is not mirrored: the decode model holds one.
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
