"""Local-directory HuggingFace checkpoints -> a quantized, device-resident LLaMA / Mistral.

Mirrors the offline half of the reference's loader: `HFLoader::from_local`, `load_config`, `load_tensors`
(single file, else the shards of `model.safetensors.index.json`), `convert_tensor_to_f32`
(crates/axonml-llm/src/hf_loader.rs:73-85, 161-277), `parse_llama_config_from_json` (:511-530) and the
module names of `load_state_dict` (crates/axonml-llm/src/llama.rs:782-822, 1040-1060, lm_head tied to the
embedding when absent).  Downloads are not mirrored.  What the reference keeps as f32 is quantised here,
tensor by tensor, by the device quantisers (`quantize_tensor`, quantize.rs:36-54) on the way in.
"""
import json
import mmap
import os
import struct

import numpy as np

from .quant import DeviceWeight, QuantError, QuantType, default_context


class ModelNotFound(QuantError):
    """LLMError::ModelNotFound (hf_loader.rs:75-77)."""


class WeightNotFound(QuantError):
    """LLMError::WeightNotFound (hf_loader.rs:286-288)."""


class UnsupportedFormat(QuantError):
    """LLMError::UnsupportedFormat (hf_loader.rs:270-273)."""


class ParseError(QuantError):
    """LLMError::ParseError."""


_DTYPES = {"F32": ("<f4", 4), "F16": ("<f2", 2), "BF16": ("<u2", 2)}


class SafetensorsFile:
    """One .safetensors file, memory-mapped: 8-byte little-endian header length, a JSON header
    {name: {dtype, shape, data_offsets}}, then the tensor bytes."""

    def __init__(self, path):
        self.path = path
        with open(path, "rb") as f:
            size = os.fstat(f.fileno()).st_size
            if size < 8:
                raise ParseError(f"{path}: too short for a safetensors header")
            self._mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        (n,) = struct.unpack("<Q", self._mm[:8])
        if n > size - 8:
            raise ParseError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(bytes(self._mm[8:8 + n]).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise ParseError(f"{path}: {e}") from None
        self._base = 8 + n
        self.entries = {}
        for name, e in header.items():
            if name == "__metadata__":
                continue
            try:
                begin, end = (int(v) for v in e["data_offsets"])
                shape, dtype = [int(s) for s in e["shape"]], str(e["dtype"])
            except (KeyError, TypeError, ValueError) as err:
                raise ParseError(f"{path}: entry {name}: {err}") from None
            if begin > end or self._base + end > size:
                raise ParseError(f"{path}: entry {name}: data offsets outside the file")
            self.entries[name] = (dtype, shape, begin, end)

    def names(self):
        return list(self.entries)

    def tensor_f32(self, name):
        """convert_tensor_to_f32 (hf_loader.rs:236-277): F32 as is, F16 and BF16 widened exactly."""
        dtype, shape, begin, end = self.entries[name]
        if dtype not in _DTYPES:
            raise UnsupportedFormat(f"Unsupported tensor dtype: {dtype}")
        np_dtype, width = _DTYPES[dtype]
        numel = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if end - begin != numel * width:
            raise ParseError(f"{self.path}: entry {name}: {end - begin} bytes for shape {shape} of {dtype}")
        raw = np.frombuffer(self._mm, dtype=np_dtype, count=numel, offset=self._base + begin)
        if dtype == "F32":
            out = raw.astype(np.float32)
        elif dtype == "F16":
            out = raw.astype(np.float32)
        else:
            out = (raw.astype(np.uint32) << 16).view(np.float32)
        return out.reshape(shape)


class HFLoader:
    """HFLoader::from_local: a directory with config.json and model.safetensors (or its shards)."""

    def __init__(self, path):
        if not os.path.isdir(path):
            raise ModelNotFound(path)
        self.path = path
        self._files, self._where = [], {}

    @classmethod
    def from_local(cls, path):
        return cls(path)

    def load_config(self):
        p = os.path.join(self.path, "config.json")
        try:
            with open(p) as f:
                return json.load(f)
        except OSError as e:
            raise ModelNotFound(f"{p}: {e}") from None
        except json.JSONDecodeError as e:
            raise ParseError(f"{p}: {e}") from None

    def load_tensors(self):
        single = os.path.join(self.path, "model.safetensors")
        if os.path.exists(single):
            shards = ["model.safetensors"]
        else:
            idx = os.path.join(self.path, "model.safetensors.index.json")
            try:
                with open(idx) as f:
                    weight_map = json.load(f)["weight_map"]
                shards = sorted(set(str(v) for v in weight_map.values()))
            except OSError as e:
                raise ModelNotFound(f"{idx}: {e}") from None
            except (json.JSONDecodeError, KeyError, AttributeError, TypeError):
                raise ParseError("Invalid index file") from None
        for shard in shards:
            f = SafetensorsFile(os.path.join(self.path, shard))
            self._files.append(f)
            for name in f.names():
                self._where[name] = f
        return len(self._where)

    def has(self, name):
        return name in self._where

    def get_tensor(self, name):
        if name not in self._where:
            raise WeightNotFound(name)
        return self._where[name].tensor_f32(name)


def parse_llama_config_from_json(cfg, max_position_embeddings=None):
    """parse_llama_config_from_json (hf_loader.rs:511-530) with its defaults; the same keys serve Mistral
    (parse_mistral_config, :557-572).  The position limit sizes the KV cache, so a caller may lower it."""
    heads = int(cfg.get("num_attention_heads", 32))
    hidden = int(cfg.get("hidden_size", 4096))
    return dict(vocab_size=int(cfg.get("vocab_size", 32000)), hidden_size=hidden,
                intermediate_size=int(cfg.get("intermediate_size", 11008)),
                num_hidden_layers=int(cfg.get("num_hidden_layers", 32)), num_attention_heads=heads,
                num_key_value_heads=int(cfg.get("num_key_value_heads") or heads),
                head_dim=int(cfg.get("head_dim") or hidden // heads),
                max_position_embeddings=int(max_position_embeddings or cfg.get("max_position_embeddings", 4096)),
                rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-5)), rope_theta=float(cfg.get("rope_theta", 10000.0)),
                sliding_window=int(cfg.get("sliding_window") or 0))  # Mistral's window (parse_mistral_config, :557-572); none for LLaMA


_PROJ = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
         "gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj"}


def set_embedding(model, emb):
    """The embedding table as the reference holds it, f32 (embedding.rs:103-146).  A table whose values all fit f16 exactly
    (an F16 checkpoint) goes to the device as f16: the same rows come out, at half the memory."""
    emb = np.ascontiguousarray(emb, dtype=np.float32)
    with np.errstate(over="ignore"):
        half = emb.astype(np.float16)
    if np.array_equal(half.astype(np.float32), emb):
        model.set_embedding_f16(half.view(np.uint16))
    else:
        model.set_embedding_f32(emb)


def load_llama(path, quant_type=QuantType.Q4_K, ctx=None, max_position_embeddings=None):
    """Directory -> QuantizedLlama: every linear quantised to `quant_type` on the device as it is read."""
    from .decode import QuantizedLlama

    ctx = ctx or default_context()
    loader = HFLoader.from_local(path)
    cfg = parse_llama_config_from_json(loader.load_config(), max_position_embeddings)
    loader.load_tensors()

    def get(*names):  # load_state_dict accepts names with and without the "model." prefix (llama.rs:790-806)
        for n in names:
            if loader.has(n):
                return loader.get_tensor(n)
        raise WeightNotFound(names[0])

    model = QuantizedLlama(ctx, **cfg)
    emb = get("model.embed_tokens.weight", "embed_tokens.weight")
    set_embedding(model, emb)

    def linear(layer, which, w):
        dw = DeviceWeight.quantize(w, quant_type, ctx)
        try:
            model.set_linear(layer, which, dw)
        finally:
            dw.free()

    for i in range(cfg["num_hidden_layers"]):
        pre = (f"model.layers.{i}", f"layers.{i}")
        model.set_norm(i, 0, get(*(f"{p}.input_layernorm.weight" for p in pre)))
        model.set_norm(i, 1, get(*(f"{p}.post_attention_layernorm.weight" for p in pre)))
        for which, stem in _PROJ.items():
            linear(i, which, get(*(f"{p}.{stem}.weight" for p in pre)))
    model.set_norm(-1, 0, get("model.norm.weight", "norm.weight"))
    linear(-1, "q", loader.get_tensor("lm_head.weight") if loader.has("lm_head.weight") else emb)  # tied (llama.rs:1046-1056)
    return model
