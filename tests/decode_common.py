"""Shared builders for the decode tests: a small random model as plain arrays, loaded into the CPU
oracle, the GPU model, or the independent numpy float64 forward below."""
import numpy as np

import oracle as o

LIN_SHAPES = lambda c: {  # noqa: E731
    "q": (c["num_heads"] * c["head_dim"], c["hidden_size"]),
    "k": (c["num_kv_heads"] * c["head_dim"], c["hidden_size"]),
    "v": (c["num_kv_heads"] * c["head_dim"], c["hidden_size"]),
    "o": (c["hidden_size"], c["num_heads"] * c["head_dim"]),
    "gate": (c["intermediate_size"], c["hidden_size"]),
    "up": (c["intermediate_size"], c["hidden_size"]),
    "down": (c["hidden_size"], c["intermediate_size"]),
}
LIN_ID = {"q": 0, "k": 1, "v": 2, "o": 3, "gate": 4, "up": 5, "down": 6}


def tiny_config(**over):
    c = dict(vocab_size=320, hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4, num_kv_heads=2,
             head_dim=64, max_seq_len=48, rms_norm_eps=1e-5, rope_theta=10000.0, sliding_window=0)
    c.update(over)
    return c


def random_weights(c, seed, qtype=o.Q4_K, std=0.06):
    rng = np.random.default_rng(seed)
    w = {"emb": (rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.7).astype(np.float16).view(np.uint16),
         "final_norm": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32), "layers": [], "qtype": qtype}
    for _ in range(c["num_layers"]):
        L = {"norm0": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32),
             "norm1": (1.0 + 0.1 * rng.standard_normal(c["hidden_size"])).astype(np.float32)}
        for name, (n, k) in LIN_SHAPES(c).items():
            L[name] = o.quantize(qtype, (rng.standard_normal((n, k)) * std).astype(np.float32))
        w["layers"].append(L)
    w["head"] = o.quantize(qtype, (rng.standard_normal((c["vocab_size"], c["hidden_size"])) * std).astype(np.float32))
    return w


def load_oracle(c, w):
    m = o.DecodeModel(**c)
    m.set_embedding_f16(w["emb"])
    m.set_norm(-1, 0, w["final_norm"])
    types = w.get("types", {})  # (layer, name) -> type of the linears that differ from w["qtype"]
    for l, L in enumerate(w["layers"]):
        m.set_norm(l, 0, L["norm0"])
        m.set_norm(l, 1, L["norm1"])
        for name in LIN_ID:
            m.set_linear(l, LIN_ID[name], types.get((l, name), w["qtype"]), L[name])
    m.set_linear(-1, 0, types.get((-1, "head"), w["qtype"]), w["head"])
    return m


def load_gpu(ctx, c, w):
    from axonml_amd import quant as q
    from axonml_amd.decode import QuantizedLlama

    m = QuantizedLlama(ctx, vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
                       intermediate_size=c["intermediate_size"], num_hidden_layers=c["num_layers"],
                       num_attention_heads=c["num_heads"], num_key_value_heads=c["num_kv_heads"], head_dim=c["head_dim"],
                       max_position_embeddings=c["max_seq_len"], rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"],
                       sliding_window=c.get("sliding_window", 0))
    m.set_embedding_f16(w["emb"])
    m.set_norm(-1, 0, w["final_norm"])
    shapes = LIN_SHAPES(c)
    types = w.get("types", {})
    for l, L in enumerate(w["layers"]):
        m.set_norm(l, 0, L["norm0"])
        m.set_norm(l, 1, L["norm1"])
        for name, (n, k) in shapes.items():
            m.set_linear(l, name, q.QuantizedTensor([n, k], types.get((l, name), w["qtype"]), L[name]))
    m.set_linear(-1, "q", q.QuantizedTensor([c["vocab_size"], c["hidden_size"]], types.get((-1, "head"), w["qtype"]), w["head"]))
    return m


def requantize(c, w, changes, seed):
    """Replaces the linears named in `changes` ({(layer, name): type}; (-1, "head") is the lm_head) by fresh random
    weights of that block type and records the types in w["types"] for the loaders above."""
    rng = np.random.default_rng(seed)
    shapes = dict(LIN_SHAPES(c), head=(c["vocab_size"], c["hidden_size"]))
    for (l, name), t in changes.items():
        n, k = shapes[name]
        packed = o.quantize(t, (rng.standard_normal((n, k)) * 0.06).astype(np.float32))
        if l < 0:
            w["head"] = packed
        else:
            w["layers"][l][name] = packed
    w.setdefault("types", {}).update(changes)
    return w


class NumpyDecoder:
    """Independent float64 forward from the textbook formulas (RMSNorm, half-split RoPE, causal GQA
    softmax attention over an f16-rounded cache, SwiGLU); shares only the dequantised weights."""

    def __init__(self, c, w):
        self.c = c
        deq = lambda p, shp: o.dequantize(w["qtype"], p, shp[0] * shp[1]).reshape(shp).astype(np.float64)  # noqa: E731
        shapes = LIN_SHAPES(c)
        self.emb = w["emb"].view(np.float16).astype(np.float64)
        self.layers = [{**{n: deq(L[n], shapes[n]) for n in shapes}, "norm0": L["norm0"].astype(np.float64),
                        "norm1": L["norm1"].astype(np.float64)} for L in w["layers"]]
        self.final_norm = w["final_norm"].astype(np.float64)
        self.head = deq(w["head"], (c["vocab_size"], c["hidden_size"]))
        self.k = [[] for _ in w["layers"]]
        self.v = [[] for _ in w["layers"]]

    def _norm(self, x, w):
        return x / np.sqrt(np.mean(x * x) + self.c["rms_norm_eps"]) * w

    def _rope(self, x, pos):
        d = self.c["head_dim"]
        x = x.reshape(-1, d).copy()
        i = np.arange(d // 2)
        ang = pos * (1.0 / np.float32(self.c["rope_theta"]) ** (2.0 * i / d))
        c_, s_ = np.cos(ang), np.sin(ang)
        a, b = x[:, :d // 2].copy(), x[:, d // 2:].copy()
        x[:, :d // 2] = a * c_ - b * s_
        x[:, d // 2:] = a * s_ + b * c_
        return x

    def forward(self, token, pos):
        c = self.c
        d, nh, nkv = c["head_dim"], c["num_heads"], c["num_kv_heads"]
        h = self.emb[token].copy()
        for l, L in enumerate(self.layers):
            xn = self._norm(h, L["norm0"])
            q = self._rope(L["q"] @ xn, pos)
            k = self._rope(L["k"] @ xn, pos)
            v = (L["v"] @ xn).reshape(nkv, d)
            self.k[l].append(k.astype(np.float16).astype(np.float64))
            self.v[l].append(v.astype(np.float16).astype(np.float64))
            win = c.get("sliding_window", 0)
            first = max(0, len(self.k[l]) - win) if win else 0  # Mistral: the last `win` positions only
            K = np.stack(self.k[l][first:], 1)  # [nkv, T, d]
            V = np.stack(self.v[l][first:], 1)
            out = np.zeros((nh, d))
            for hd in range(nh):
                kv = hd // (nh // nkv)
                s = K[kv] @ q[hd] / np.sqrt(d)
                p = np.exp(s - s.max())
                out[hd] = (p / p.sum()) @ V[kv]
            h = h + L["o"] @ out.reshape(-1)
            xn = self._norm(h, L["norm1"])
            g = L["gate"] @ xn
            h = h + L["down"] @ (g / (1.0 + np.exp(-g)) * (L["up"] @ xn))
        return self.head @ self._norm(h, self.final_norm)
