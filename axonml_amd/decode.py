"""Host-side mirror of the reference's LLaMA/Mistral decode loop over the axq C ABI.

`QuantizedLlama` plays the part of LLaMAForCausalLM (crates/axonml-llm/src/llama.rs:834-1100) for one
sequence: `forward_with_cache`-style single-token steps and greedy `generate`, with every linear a
quantized, device-resident weight.  Config field names follow LLaMAConfig / MistralConfig.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import MEM_HOST
from .quant import DeviceWeight, QuantType, ShapeMismatch, default_context

LINEARS = {"q": 0, "k": 1, "v": 2, "o": 3, "gate": 4, "up": 5, "down": 6}


def mistral_7b_config(max_position_embeddings=640):
    """MistralConfig::mistral_7b (crates/axonml-llm/src/mistral.rs:56-70), context capped to the cache size."""
    return dict(vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                max_position_embeddings=max_position_embeddings, rms_norm_eps=1e-5, rope_theta=10000.0, sliding_window=4096)


class QuantizedLlama:
    def __init__(self, ctx=None, **cfg):
        self.ctx = ctx or default_context()
        self.cfg = _lib.ModelConfig(**cfg)
        h = C.c_void_p()
        self.ctx.check(self.ctx.lib.axq_model_create(self.ctx.handle, C.byref(self.cfg), C.byref(h)))
        self.handle = h

    # ---- weights
    def set_embedding_f16(self, table_bits):
        t = np.ascontiguousarray(table_bits, dtype=np.uint16)
        if t.size != self.cfg.vocab_size * self.cfg.hidden_size:
            raise ShapeMismatch(f"Shape mismatch: embedding table of {t.size} elements, expected vocab_size * hidden_size = "
                                f"{self.cfg.vocab_size} * {self.cfg.hidden_size}")
        self.ctx.check(self.ctx.lib.axq_model_set_embedding_f16(self.handle, t.ctypes.data, MEM_HOST))

    def set_embedding_f32(self, table):
        """The embedding table in f32, as the reference keeps it (embedding.rs:103-146)."""
        t = np.ascontiguousarray(table, dtype=np.float32)
        if t.size != self.cfg.vocab_size * self.cfg.hidden_size:
            raise ShapeMismatch(f"Shape mismatch: embedding table of {t.size} elements, expected vocab_size * hidden_size = "
                                f"{self.cfg.vocab_size} * {self.cfg.hidden_size}")
        self.ctx.check(self.ctx.lib.axq_model_set_embedding_f32(self.handle, t.ctypes.data, MEM_HOST))

    def set_norm(self, layer, which, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        if w.size != self.cfg.hidden_size:  # the library copies hidden_size floats from this pointer
            raise ShapeMismatch(f"Shape mismatch: norm weight of {w.size} elements, expected hidden_size = {self.cfg.hidden_size}")
        self.ctx.check(self.ctx.lib.axq_model_set_norm(self.handle, layer, which, w.ctypes.data, MEM_HOST))

    def set_linear(self, layer, name, weight):
        """weight: QuantizedTensor or DeviceWeight of the linear's [out, in] shape; layer -1 = lm_head."""
        if name not in LINEARS:
            raise KeyError(f"unknown linear {name!r}: one of {sorted(LINEARS)}")
        dw = weight if isinstance(weight, DeviceWeight) else DeviceWeight.upload(weight, self.ctx)
        try:
            self.ctx.check(self.ctx.lib.axq_model_set_linear(self.handle, layer, LINEARS[name], dw.handle))
        finally:
            if dw is not weight:
                dw.free()

    def random_init(self, quant_type=QuantType.Q4_K, std=0.02, seed=1):
        self.ctx.check(self.ctx.lib.axq_model_random_init(self.handle, int(quant_type), std, seed))

    def set_sampling(self, config=None, seed=0):
        """Next tokens by a GenerationConfig (temperature, top-k, top-p, repetition penalty over every token fed so
        far, draws from (seed, position)) instead of the plain argmax; None goes back to greedy."""
        cfg = config.to_c() if config is not None else None
        self.ctx.check(self.ctx.lib.axq_model_set_sampling(self.handle, C.byref(cfg) if cfg is not None else None, int(seed)))

    # ---- stepping
    def reset(self):
        self.ctx.check(self.ctx.lib.axq_model_reset(self.handle))

    def seq_len(self):
        return self.ctx.lib.axq_model_seq_len(self.handle)

    def forward(self, token, want_logits=True):
        logits = np.empty(self.cfg.vocab_size, dtype=np.float32) if want_logits else None
        nxt = C.c_int32()
        self.ctx.check(self.ctx.lib.axq_model_forward(self.handle, int(token), logits.ctypes.data if want_logits else None,
                                                      C.byref(nxt)))
        return nxt.value, logits

    def forward_tokens(self, tokens, want_logits=True):
        """forward_with_cache on several tokens (a prompt): the last position's next token and logits."""
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.cfg.vocab_size, dtype=np.float32) if want_logits else None
        nxt = C.c_int32()
        self.ctx.check(self.ctx.lib.axq_model_forward_tokens(self.handle, t.ctypes.data, t.size,
                                                             logits.ctypes.data if want_logits else None, C.byref(nxt)))
        return nxt.value, logits

    def set_batch(self, n_seq):
        """Caches and positions for n_seq sequences side by side (1..64); starts all of them afresh."""
        self.ctx.check(self.ctx.lib.axq_model_set_batch(self.handle, int(n_seq)))

    def batch(self):
        return self.ctx.lib.axq_model_batch(self.handle)

    def seq_len_of(self, seq):
        return self.ctx.lib.axq_model_seq_len_of(self.handle, int(seq))

    def copy_sequence(self, src, dst):
        """Sequence dst becomes a copy of sequence src (cache, history, position)."""
        self.ctx.check(self.ctx.lib.axq_model_copy_sequence(self.handle, int(src), int(dst)))

    def forward_batch(self, tokens, want_logits=True):
        """One token of every sequence: (next tokens [n_seq], logits [n_seq, vocab])."""
        n = self.batch()
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        if t.shape != (n,):
            raise ValueError(f"{n} tokens wanted, one per sequence")
        logits = np.empty((n, self.cfg.vocab_size), dtype=np.float32) if want_logits else None
        nxt = np.empty(n, dtype=np.int32)
        self.ctx.check(self.ctx.lib.axq_model_forward_batch(self.handle, t.ctypes.data, logits.ctypes.data if want_logits else None,
                                                            nxt.ctypes.data))
        return nxt, logits

    def generate_batch(self, prompts, max_new_tokens):
        """prompts: n_seq token lists of any lengths -> (ids [n_seq, max_new_tokens], prompt ms, generation ms)."""
        n = self.batch()
        if len(prompts) != n:
            raise ValueError(f"{n} prompts wanted, one per sequence")
        flat = np.ascontiguousarray(np.concatenate([np.asarray(p, dtype=np.int32).reshape(-1) for p in prompts]), dtype=np.int32)
        offsets = np.zeros(n + 1, dtype=np.int32)
        offsets[1:] = np.cumsum([len(p) for p in prompts])
        out = np.empty((n, max_new_tokens), dtype=np.int32)
        pre, dec = C.c_float(), C.c_float()
        self.ctx.check(self.ctx.lib.axq_model_generate_batch(self.handle, flat.ctypes.data, offsets.ctypes.data, max_new_tokens,
                                                             out.ctypes.data, C.byref(pre), C.byref(dec)))
        return out, pre.value, dec.value

    def truncate(self, n_positions):
        """Rewind the cache to its first n_positions."""
        self.ctx.check(self.ctx.lib.axq_model_truncate(self.handle, int(n_positions)))

    def hidden(self):
        out = np.empty(self.cfg.hidden_size, dtype=np.float32)
        self.ctx.check(self.ctx.lib.axq_model_read_hidden(self.handle, out.ctypes.data))
        return out

    def kv(self, layer, which):
        c = self.cfg
        out = np.empty((c.num_key_value_heads, c.max_position_embeddings, c.head_dim), dtype=np.uint16)
        self.ctx.check(self.ctx.lib.axq_model_read_kv(self.handle, layer, which, out.ctypes.data))
        return out

    def generate(self, prompt, max_new_tokens):
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(max_new_tokens, dtype=np.int32)
        pre, dec = C.c_float(), C.c_float()
        self.ctx.check(self.ctx.lib.axq_model_generate(self.handle, p.ctypes.data, p.size, max_new_tokens, out.ctypes.data,
                                                       C.byref(pre), C.byref(dec)))
        return out, pre.value, dec.value

    def close(self):
        if self.handle:
            self.ctx.lib.axq_model_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _bench_q4_k_m_mix(ctx, m, cfg, prompt, new_tokens, weight_elems, mean_ctx, log):
    """The same model with the block types of llama.cpp's Q4_K_M recipe: attn_v and ffn_down of half the layers
    (use_more_bits: the first and last eighth and every third between) and the output matrix in Q6_K, the rest Q4_K.
    A v of another type than q and k is multiplied apart, one more GEMV in those layers."""
    from ._lib import MEM_DEVICE
    lib, L = ctx.lib, cfg["num_hidden_layers"]
    more = [l for l in range(L) if l < L // 8 or l >= 7 * L // 8 or (l - L // 8) % 3 == 2]
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    kv = cfg["num_key_value_heads"] * cfg["head_dim"]
    f = ctx.malloc(max(V * H, H * I) * 4)
    seed, q6_elems = 1000, 0
    for l, name, n, k in [(l, nm, n, k) for l in more for nm, n, k in (("v", kv, H), ("down", H, I))] + [(-1, "q", V, H)]:
        seed += 1
        ctx.check(lib.axq_fill_normal_f32(ctx.handle, f, n * k, 0.0, 0.02, 0.0, 0.0, seed))
        h = C.c_void_p()
        ctx.check(lib.axq_weight_quantize(ctx.handle, int(QuantType.Q6_K), n, k, f, MEM_DEVICE, C.byref(h)))
        dw = DeviceWeight(ctx, h, QuantType.Q6_K, n, k)
        m.set_linear(l, name, dw)
        dw.free()
        q6_elems += n * k
    ctx.free(f)
    m.reset()
    m.generate(prompt, 4)
    m.reset()
    _, pre_ms, dec_ms = m.generate(prompt, new_tokens)
    steps = new_tokens - 1
    tok_s = steps / (dec_ms * 1e-3)
    nbytes = (weight_elems - q6_elems) * 0.5625 + q6_elems * 210 / 256 + 131072 * mean_ctx + 131072
    log(f"  Q4_K_M mix ({len(more)} layers with attn_v and ffn_down in Q6_K, output in Q6_K): {tok_s:.1f} tok/s, "
        f"{nbytes * tok_s / 1e9:.0f} GB/s")
    return {"q4_k_m_mix_tokens_per_s": tok_s, "q4_k_m_mix_algorithmic_bytes_per_token": nbytes,
            "q4_k_m_mix_gbps": nbytes * tok_s / 1e9, "q4_k_m_mix_prefill_tokens_per_s": len(prompt) / (pre_ms * 1e-3),
            "q4_k_m_mix_q6_k_layers": len(more)}


def bench_7b(ctx, log=print, prompt_len=512, new_tokens=128, one_sequence_only=False):
    """Decode benchmark: Mistral-7B shape, random init, all linears Q4_K, f16 KV cache; greedy, sampled, and several
    sequences side by side (one_sequence_only: the greedy single-sequence run alone, for kernel profiles)."""
    cfg = mistral_7b_config(prompt_len + new_tokens)
    m = QuantizedLlama(ctx, **cfg)
    m.random_init(QuantType.Q4_K, 0.02, 1)
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, cfg["vocab_size"], size=prompt_len, dtype=np.int32)
    m.generate(prompt, 4)  # warm-up: graph capture, scratch buffers of the prompt path, first touch
    m.reset()
    out, pre_ms, dec_ms = m.generate(prompt, new_tokens)
    steps = new_tokens - 1
    weights = 32 * (2 * 4096 * 4096 + 2 * 1024 * 4096 + 3 * 14336 * 4096) + 32000 * 4096
    mean_ctx = prompt_len + new_tokens / 2
    bytes_per_token = weights * 0.5625 + 131072 * mean_ctx + 131072
    tok_s = steps / (dec_ms * 1e-3)
    res = {"model": "Mistral-7B shape, random init, Q4_K linears, f16 KV cache", "prompt_tokens": prompt_len,
           "generated_tokens": new_tokens, "prefill_ms": pre_ms, "prefill_tokens_per_s": prompt_len / (pre_ms * 1e-3),
           "decode_ms": dec_ms, "decode_steps_timed": steps, "tokens_per_s": tok_s, "ms_per_token": dec_ms / steps,
           "algorithmic_bytes_per_token": bytes_per_token, "gbps": bytes_per_token * tok_s / 1e9,
           "frac_of_hbm_peak": bytes_per_token * tok_s / 8e12, "distinct_generated_ids": int(len(set(out.tolist())))}
    log(f"  decode 7B-shape: {tok_s:.1f} tok/s ({res['ms_per_token']:.3f} ms/token, {res['gbps']:.0f} GB/s), "
        f"prefill {res['prefill_tokens_per_s']:.0f} tok/s")
    if one_sequence_only:
        m.close()
        return res
    # the same with the sampler in the loop (temperature 0.8, top-k 40, top-p 0.9, repetition penalty 1.1)
    from .generation import GenerationConfig

    m.reset()
    m.set_sampling(GenerationConfig(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.1), seed=7)
    m.generate(prompt[:8], 4)
    m.reset()
    _, _, dec_s = m.generate(prompt, new_tokens)
    res["sampled_tokens_per_s"] = steps / (dec_s * 1e-3)
    res["sampler_us_per_token"] = (dec_s - dec_ms) / steps * 1e3
    log(f"  with top-k/top-p sampling: {res['sampled_tokens_per_s']:.1f} tok/s (sampler {res['sampler_us_per_token']:.0f} us per token)")
    # eight sequences side by side, greedy: one pass over the weights per step serves all of them
    m.set_sampling(None)
    for n_seq in (2, 4, 8):
        m.set_batch(n_seq)
        prompts = [rng.integers(0, cfg["vocab_size"], size=prompt_len, dtype=np.int32) for _ in range(n_seq)]
        m.generate_batch(prompts, 4)
        _, pre_b, dec_b = m.generate_batch(prompts, new_tokens)
        res[f"batch{n_seq}_tokens_per_s"] = n_seq * new_tokens / (dec_b * 1e-3)
        res[f"batch{n_seq}_ms_per_step"] = dec_b / new_tokens
        res[f"batch{n_seq}_prefill_tokens_per_s"] = n_seq * (prompt_len - 1) / (pre_b * 1e-3)
        log(f"  {n_seq} sequences: {res[f'batch{n_seq}_tokens_per_s']:.0f} tok/s in all ({res[f'batch{n_seq}_ms_per_step']:.3f} ms per step), "
            f"prompts {res[f'batch{n_seq}_prefill_tokens_per_s']:.0f} tok/s")
    m.set_sampling(GenerationConfig(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.1), seed=7)
    m.generate_batch(prompts, 4)
    _, _, dec_bs = m.generate_batch(prompts, new_tokens)
    res["batch8_sampled_tokens_per_s"] = 8 * new_tokens / (dec_bs * 1e-3)
    log(f"  8 sequences with top-k/top-p sampling: {res['batch8_sampled_tokens_per_s']:.0f} tok/s in all")
    # 64 sequences: the linears of a step are GEMMs on f32 rows
    m.set_sampling(None)
    m.set_batch(64)
    prompts = [rng.integers(0, cfg["vocab_size"], size=prompt_len, dtype=np.int32) for _ in range(64)]
    m.generate_batch([p[:8] for p in prompts], 4)
    _, pre_b, dec_b = m.generate_batch(prompts, new_tokens)
    res["batch64_tokens_per_s"] = 64 * new_tokens / (dec_b * 1e-3)
    res["batch64_ms_per_step"] = dec_b / new_tokens
    log(f"  64 sequences: {res['batch64_tokens_per_s']:.0f} tok/s in all ({res['batch64_ms_per_step']:.3f} ms per step)")
    m.set_batch(1)
    res.update(_bench_q4_k_m_mix(ctx, m, cfg, prompt, new_tokens, weights, mean_ctx, log))  # last: it changes the weights
    m.close()
    return res
