"""Local HuggingFace checkpoints: the safetensors reader against files written by the `safetensors`
package and by hand (BF16), the config defaults of the reference, and (GPU) a tiny LLaMA quantised on
load against the CPU decode oracle fed with the oracle's quantisation of the same f32 weights."""
import json
import struct

import numpy as np
import pytest

import oracle as o
from axonml_amd import hf_loader as hf
from axonml_amd import quant as q


def _write_safetensors(path, tensors):
    """tensors: name -> (dtype string, shape, raw bytes).  The format's own layout, written by hand."""
    header, blobs, pos = {}, [], 0
    for name, (dtype, shape, raw) in tensors.items():
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [pos, pos + len(raw)]}
        blobs.append(raw)
        pos += len(raw)
    header["__metadata__"] = {"format": "pt"}
    h = json.dumps(header).encode()
    h += b" " * (-len(h) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"".join(blobs))


def _bf16_bits(x):
    return np.array([o.lib().axo_f32_to_bf16(float(v)) for v in np.asarray(x, np.float32).reshape(-1)], dtype=np.uint16)


def test_reader_against_the_safetensors_package(tmp_path):
    from safetensors.numpy import save_file

    rng = np.random.default_rng(0)
    a = rng.standard_normal((3, 5)).astype(np.float32)
    b = rng.standard_normal((7,)).astype(np.float16)
    p = str(tmp_path / "m.safetensors")
    save_file({"a": a, "b": b}, p)
    f = hf.SafetensorsFile(p)
    assert sorted(f.names()) == ["a", "b"]
    assert np.array_equal(f.tensor_f32("a"), a) and f.tensor_f32("a").dtype == np.float32
    assert np.array_equal(f.tensor_f32("b"), b.astype(np.float32))  # f16 widens exactly (hf_loader.rs:252-260)


def test_bf16_widens_exactly_and_other_dtypes_are_refused(tmp_path):
    vals = np.array([1.0, -2.5, 3.140625, 1e-3, 65536.0, -0.0], dtype=np.float32)
    bits = _bf16_bits(vals)
    p = str(tmp_path / "m.safetensors")
    _write_safetensors(p, {"w": ("BF16", (2, 3), bits.tobytes()), "i": ("I64", (1,), b"\0" * 8)})
    f = hf.SafetensorsFile(p)
    want = (bits.astype(np.uint32) << 16).view(np.float32).reshape(2, 3)  # half::bf16::to_f32: the bits, shifted
    assert np.array_equal(f.tensor_f32("w"), want)
    assert np.array_equal(want.reshape(-1)[:3], vals[:3])  # representable values come back as they were
    with pytest.raises(hf.UnsupportedFormat, match="I64"):
        f.tensor_f32("i")


def test_malformed_files(tmp_path):
    p = tmp_path / "m.safetensors"
    p.write_bytes(b"\1\2\3")
    with pytest.raises(hf.ParseError):
        hf.SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(hf.ParseError, match="exceeds"):
        hf.SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 2) + b"{x")
    with pytest.raises(hf.ParseError):
        hf.SafetensorsFile(str(p))
    _write_safetensors(str(p), {"w": ("F32", (4,), b"\0" * 8)})  # 8 bytes for four f32
    with pytest.raises(hf.ParseError, match="bytes for shape"):
        hf.SafetensorsFile(str(p)).tensor_f32("w")
    with pytest.raises(hf.ModelNotFound):
        hf.HFLoader.from_local(str(tmp_path / "missing"))
    d = tmp_path / "empty"
    d.mkdir()
    with pytest.raises(hf.ModelNotFound):
        hf.HFLoader.from_local(str(d)).load_tensors()
    (d / "model.safetensors.index.json").write_text("{}")
    with pytest.raises(hf.ParseError, match="Invalid index file"):
        hf.HFLoader.from_local(str(d)).load_tensors()


def test_config_defaults_follow_the_reference():
    # parse_llama_config_from_json (hf_loader.rs:511-530): every key optional, LLaMA-2-7B defaults
    c = hf.parse_llama_config_from_json({})
    assert c == dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                     num_key_value_heads=32, head_dim=128, max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=10000.0,
                     sliding_window=0)
    c = hf.parse_llama_config_from_json({"num_attention_heads": 8, "hidden_size": 512, "num_key_value_heads": 2, "rope_theta": 1e6},
                                        max_position_embeddings=64)
    assert c["num_key_value_heads"] == 2 and c["head_dim"] == 64 and c["max_position_embeddings"] == 64 and c["rope_theta"] == 1e6
    assert hf.parse_llama_config_from_json({"num_attention_heads": 8})["num_key_value_heads"] == 8  # falls back to the head count
    assert hf.parse_llama_config_from_json({"sliding_window": 4096})["sliding_window"] == 4096  # Mistral's config.json
    assert hf.parse_llama_config_from_json({"sliding_window": None})["sliding_window"] == 0


def _tiny_checkpoint(tmp_path, c, seed, sharded, tied, prefix="model."):
    """f32 weights of a tiny LLaMA as a checkpoint directory (a mix of F32, F16 and BF16 tensors), and the
    same weights as the loader will see them after widening."""
    from tests.decode_common import LIN_SHAPES

    rng = np.random.default_rng(seed)
    seen, files = {}, [{}, {}]

    def put(name, arr, dtype, shard):
        arr = np.asarray(arr, np.float32)
        if dtype == "F32":
            raw, back = arr.tobytes(), arr
        elif dtype == "F16":
            h = arr.astype(np.float16)
            raw, back = h.tobytes(), h.astype(np.float32)
        else:
            bits = _bf16_bits(arr).reshape(arr.shape)
            raw, back = bits.tobytes(), (bits.astype(np.uint32) << 16).view(np.float32)
        files[shard if sharded else 0][name] = (dtype, arr.shape, raw)
        seen[name] = back

    # tied checkpoints carry an F32 table whose values do not fit f16 (the loader must keep them), the others an F16 table
    put(f"{prefix}embed_tokens.weight", rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.7, "F32" if tied else "F16", 0)
    stems = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
             "gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj"}
    for i in range(c["num_layers"]):
        put(f"{prefix}layers.{i}.input_layernorm.weight", 1.0 + 0.1 * rng.standard_normal(c["hidden_size"]), "F32", i % 2)
        put(f"{prefix}layers.{i}.post_attention_layernorm.weight", 1.0 + 0.1 * rng.standard_normal(c["hidden_size"]), "BF16", i % 2)
        for j, (name, shape) in enumerate(LIN_SHAPES(c).items()):
            put(f"{prefix}layers.{i}.{stems[name]}.weight", rng.standard_normal(shape) * 0.06, ("F32", "F16", "BF16")[j % 3], i % 2)
    put(f"{prefix}norm.weight", 1.0 + 0.1 * rng.standard_normal(c["hidden_size"]), "F32", 1)
    if not tied:
        put("lm_head.weight", rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.06, "BF16", 1)
    d = tmp_path / f"ckpt{seed}"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(dict(
        vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
        num_hidden_layers=c["num_layers"], num_attention_heads=c["num_heads"], num_key_value_heads=c["num_kv_heads"],
        max_position_embeddings=c["max_seq_len"], rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"])))
    if sharded:
        names = ["model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"]
        for fn, t in zip(names, files):
            _write_safetensors(str(d / fn), t)
        (d / "model.safetensors.index.json").write_text(json.dumps(
            {"weight_map": {k: fn for fn, t in zip(names, files) for k in t}}))
    else:
        _write_safetensors(str(d / "model.safetensors"), files[0])
    return str(d), seen, stems


@pytest.mark.gpu
@pytest.mark.parametrize("qtype,sharded,tied,prefix", [(o.Q4_K, False, False, "model."), (o.Q8_0, True, True, "model."),
                                                      (o.Q4_0, True, False, "")])
def test_llama_quantised_on_load_decodes_like_the_oracle(ctx, tmp_path, qtype, sharded, tied, prefix):
    from tests.decode_common import LIN_ID, LIN_SHAPES, tiny_config
    from tests.util import DECODE_FLOOR, DECODE_RTOL, max_rel_err

    c = tiny_config()
    path, seen, stems = _tiny_checkpoint(tmp_path, c, 31 + qtype, sharded, tied, prefix)
    gpu = hf.load_llama(path, q.QuantType(qtype), ctx)
    # the oracle gets the oracle's own quantisation of the widened f32 weights (bit-exact with the device's for
    # these types, see tests/test_gpu_codecs.py), so any difference comes from the loader
    cpu = o.DecodeModel(vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
                        num_layers=c["num_layers"], num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"], head_dim=c["head_dim"],
                        max_seq_len=c["max_seq_len"], rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"])
    emb = seen[f"{prefix}embed_tokens.weight"]
    cpu.set_embedding_f32(emb)  # the reference's table is f32 (embedding.rs:103-146)
    if tied:
        assert not np.array_equal(emb.astype(np.float16).astype(np.float32), emb)
    for i in range(c["num_layers"]):
        cpu.set_norm(i, 0, seen[f"{prefix}layers.{i}.input_layernorm.weight"])
        cpu.set_norm(i, 1, seen[f"{prefix}layers.{i}.post_attention_layernorm.weight"])
        for name in LIN_SHAPES(c):
            cpu.set_linear(i, LIN_ID[name], qtype, o.quantize(qtype, seen[f"{prefix}layers.{i}.{stems[name]}.weight"]))
    cpu.set_norm(-1, 0, seen[f"{prefix}norm.weight"])
    cpu.set_linear(-1, 0, qtype, o.quantize(qtype, emb if tied else seen["lm_head.weight"]))
    tok = 9
    for pos in range(10):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.close()
    cpu.close()


@pytest.mark.gpu
def test_missing_weight_is_named(ctx, tmp_path):
    from tests.decode_common import tiny_config

    c = tiny_config(num_layers=1)
    path, _, _ = _tiny_checkpoint(tmp_path, c, 5, False, False)
    # drop one projection
    f = hf.SafetensorsFile(path + "/model.safetensors")
    keep = {n: (f.entries[n][0], f.entries[n][1], bytes(f._mm[f._base + f.entries[n][2]:f._base + f.entries[n][3]]))
            for n in f.names() if "up_proj" not in n}
    _write_safetensors(path + "/model.safetensors", keep)
    with pytest.raises(hf.WeightNotFound, match="up_proj"):
        hf.load_llama(path, q.QuantType.Q8_0, ctx)
