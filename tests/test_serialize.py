"""State dictionaries on disk: the reference's bincode / JSON layouts (checked against bytes assembled by
hand from the bincode 1.3 rules, and against the reference's own unit tests of StateDict and Format), and
the quantized entry added behind them."""
import json
import struct

import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from axonml_amd import serialize as s


def _u64(v):
    return struct.pack("<Q", v)


def _str(t):
    b = t.encode()
    return _u64(len(b)) + b


def _hand_assembled():
    """bincode::serialize(&StateDict) for one entry "w": shape [2, 3], values 1..6, requires_grad = false,
    entry metadata {"k": "v"}, dictionary metadata {"format": "x"}: field by field, as bincode 1.3 lays them out."""
    entry = (_str("w")                                              # HashMap key
             + _u64(2) + _u64(2) + _u64(3)                          # data.shape: Vec<usize>
             + _u64(6) + struct.pack("<6f", 1, 2, 3, 4, 5, 6)       # data.values: Vec<f32>
             + b"\x00"                                              # requires_grad
             + _u64(1) + _str("k") + _str("v"))                     # metadata
    return _u64(1) + entry + _u64(1) + _str("format") + _str("x")   # entries, then metadata


def _example():
    sd = s.StateDict()
    sd.insert_entry("w", s.StateDictEntry(s.TensorData([2, 3], [1, 2, 3, 4, 5, 6]), False).with_metadata("k", "v"))
    sd.set_metadata("format", "x")
    return sd


def test_native_bytes_are_bincode(tmp_path):
    p = tmp_path / "m.axonml"
    s.save_state_dict(_example(), p)
    assert p.read_bytes() == _hand_assembled()
    back = s.load_state_dict(p)
    e = back.get("w")
    assert e.data.shape == [2, 3] and e.data.values.tolist() == [1, 2, 3, 4, 5, 6]
    assert e.requires_grad is False and e.metadata == {"k": "v"} and back.get_metadata("format") == "x"
    assert back.quantized == {}
    assert np.array_equal(e.data.to_tensor(), np.arange(1, 7, dtype=np.float32).reshape(2, 3))


def test_f32_bit_patterns_survive(tmp_path):
    bits = np.array([0x7FC00001, 0xFF800000, 0x00000001, 0x80000000, 0x3DCCCCCD], dtype=np.uint32)
    sd = s.StateDict()
    sd.insert("x", s.TensorData([5], bits.view(np.float32)))
    p = tmp_path / "m.bin"
    s.save_state_dict(sd, p)
    assert np.array_equal(s.load_state_dict(p).get("x").data.values.view(np.uint32), bits)


def test_reference_unit_tests_of_state_dict_and_format():
    # state_dict.rs tests: operations, filter_prefix, strip_prefix, merge, summary
    sd = s.StateDict()
    sd.insert("linear.weight", s.TensorData([10, 5], np.zeros(50)))
    sd.insert("linear.bias", s.TensorData([5], np.zeros(5)))
    assert len(sd) == 2 and sd.total_params() == 55 and sd.contains("linear.weight") and sd.contains("linear.bias")
    assert sd.size_bytes() == 220
    sd = s.StateDict()
    for n in ("encoder.layer1.weight", "encoder.layer1.bias", "decoder.layer1.weight"):
        sd.insert(n, s.TensorData([10], np.zeros(10)))
    enc = sd.filter_prefix("encoder.")
    assert len(enc) == 2 and enc.contains("encoder.layer1.weight")
    sd = s.StateDict()
    sd.insert("model.linear.weight", s.TensorData([10], np.zeros(10)))
    assert sd.strip_prefix("model.").contains("linear.weight")
    assert sd.add_prefix("a.").contains("a.model.linear.weight")
    d1, d2 = s.StateDict(), s.StateDict()
    d1.insert("a", s.TensorData([1], [1.0]))
    d2.insert("b", s.TensorData([1], [2.0]))
    d1.merge(d2)
    assert len(d1) == 2 and d1.contains("a") and d1.contains("b")
    sd = s.StateDict()
    sd.insert("weight", s.TensorData([10, 5], np.zeros(50)))
    assert "1 entries" in sd.summary() and "50" in sd.summary()
    assert sd.remove("weight") is not None and sd.is_empty()
    # format.rs tests
    want = {"model.axonml": s.Format.Axonml, "model.bin": s.Format.Axonml, "model.json": s.Format.Json,
            "model.safetensors": s.Format.SafeTensors, "model.st": s.Format.SafeTensors, "model.unknown": s.Format.Axonml,
            "model": s.Format.Axonml, "dir.json/model": s.Format.Axonml, ".json": s.Format.Axonml}
    for name, fmt in want.items():
        assert s.detect_format(name) == fmt, name
    assert s.Format.is_binary(s.Format.Axonml) and not s.Format.is_binary(s.Format.Json) and s.Format.is_binary(s.Format.SafeTensors)
    assert s.Format.extension(s.Format.Axonml) == "axonml" and s.Format.extension(s.Format.Json) == "json"
    assert s.detect_format_from_bytes(b'{"key": "value"}') == s.Format.Json
    assert s.detect_format_from_bytes(bytes(range(8))) == s.Format.Axonml
    assert s.detect_format_from_bytes(b"abc") is None
    assert s.detect_format_from_bytes(struct.pack("<Q", 64) + b'{"a":1}  ') == s.Format.SafeTensors


def _quantized_example(seed=0):
    rng = np.random.default_rng(seed)
    sd = _example()
    sd.insert("norm.weight", s.TensorData([64], rng.standard_normal(64)))
    tensors = {}
    for name, qt, shape in (("a.weight", o.Q4_K, (8, 256)), ("b.weight", o.Q8_0, (3, 64)), ("c.weight", o.Q4_0, (5, 40)),
                            ("d.weight", o.Q5_1, (2, 32)), ("e.weight", o.F16, (7,)), ("f.weight", o.Q4_1, (1, 33))):
        w = rng.standard_normal(shape).astype(np.float32)
        tensors[name] = q.QuantizedTensor(shape, q.QuantType(qt), o.quantize(qt, w))
        sd.insert_quantized(name, tensors[name])
    return sd, tensors


@pytest.mark.parametrize("ext", ["axonml", "json"])
def test_quantized_entries_round_trip(tmp_path, ext):
    sd, tensors = _quantized_example()
    p = tmp_path / f"m.{ext}"
    s.save_state_dict(sd, p)
    back = s.load_state_dict(p)
    assert set(back.quantized) == set(tensors) and set(back.keys()) == {"w", "norm.weight"}
    for name, t in tensors.items():
        b = back.get_quantized(name)
        assert b.quant_type == t.quant_type and b.shape == t.shape and np.array_equal(b.data, t.data), name
    assert np.array_equal(back.get("norm.weight").data.values, sd.get("norm.weight").data.values)
    assert back.get("w").metadata == {"k": "v"} and back.get_metadata("format") == "x"
    assert back.quantized_bytes() == sum(t.data.size for t in tensors.values())


def test_native_file_layout_with_quantized_section(tmp_path):
    """The f32 part is the reference's file unchanged (a reader that stops after the StateDict, as
    bincode::deserialize does, sees exactly that); the section behind it is laid out as documented."""
    sd = _example()
    blocks = o.quantize(o.Q8_0, np.arange(64, dtype=np.float32).reshape(2, 32))
    sd.insert_quantized("qw", q.QuantizedTensor([2, 32], q.QuantType.Q8_0, blocks))
    p = tmp_path / "m.axonml"
    s.save_state_dict(sd, p)
    raw = p.read_bytes()
    head = _hand_assembled()
    assert raw[:len(head)] == head
    section = (_u64(1) + _str("qw") + struct.pack("<I", 0) + _u64(2) + _u64(2) + _u64(32) + _u64(68) + bytes(blocks))
    assert raw[len(head):] == section + b"AXQTENS1" + _u64(len(head))
    # what the reference's load_state_dict reads from this file: the leading StateDict, nothing else
    plain = s.StateDict()
    r = s._Reader(memoryview(raw))
    s._decode_state_dict(r, plain)
    assert r.pos == len(head) and list(plain.keys()) == ["w"]


def test_json_text_is_what_serde_reads(tmp_path):
    sd, _ = _quantized_example(1)
    p = tmp_path / "m.json"
    s.save_state_dict(sd, p)
    doc = json.loads(p.read_text())
    assert set(doc) == {"entries", "metadata", "quantized"}
    assert doc["entries"]["w"] == {"data": {"shape": [2, 3], "values": [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]}, "requires_grad": False,
                                   "metadata": {"k": "v"}}
    assert doc["quantized"]["a.weight"]["quant_type"] == "Q4_K" and len(doc["quantized"]["a.weight"]["data"]) == 8 * 144
    # shortest digits that give the f32 back
    sd2 = s.StateDict()
    sd2.insert("x", s.TensorData([3], np.array([0.1, 1e20, -2.5e-7], np.float32)))
    s.save_state_dict(sd2, p)
    assert '"values": [0.1, 1e+20, -2.5e-07]' in p.read_text()
    assert np.array_equal(s.load_state_dict(p).get("x").data.values, np.array([0.1, 1e20, -2.5e-7], np.float32))
    # a file without the extra key (what the reference writes) loads with no quantized entries
    p.write_text(json.dumps({"entries": {"w": {"data": {"shape": [1], "values": [2.0]}, "requires_grad": True}}}))
    back = s.load_state_dict(p)
    assert back.get("w").data.values.tolist() == [2.0] and back.get("w").metadata == {} and back.quantized == {}


def test_malformed_files(tmp_path):
    p = tmp_path / "m.axonml"
    head = _hand_assembled()
    for cut in (0, 7, 20, len(head) - 1):
        p.write_bytes(head[:cut])
        with pytest.raises(s.SerializeError, match="unexpected end"):
            s.load_state_dict(p)
    p.write_bytes(_u64(1 << 40))  # a count the file cannot hold
    with pytest.raises(s.SerializeError, match="unexpected end"):
        s.load_state_dict(p)
    bad_bool = bytearray(head)
    bad_bool[head.index(b"\x00" + _u64(1) + _str("k"))] = 7
    p.write_bytes(bytes(bad_bool))
    with pytest.raises(s.SerializeError, match="bool"):
        s.load_state_dict(p)
    blocks = bytes(o.quantize(o.Q8_0, np.ones((1, 32), np.float32)))

    def with_section(tag=0, shape=(1, 32), data=blocks, offset=len(head), extra=b""):
        sec = _u64(1) + _str("qw") + struct.pack("<I", tag) + _u64(len(shape)) + b"".join(_u64(v) for v in shape) + _u64(len(data)) + data
        p.write_bytes(head + sec + extra + b"AXQTENS1" + _u64(offset))

    with_section()
    assert s.load_state_dict(p).get_quantized("qw").shape == [1, 32]
    with_section(tag=99)
    with pytest.raises(s.SerializeError, match="tag 99"):
        s.load_state_dict(p)
    with_section(shape=(2, 32))
    with pytest.raises(q.DataLengthMismatch):  # QuantizedTensor::from_bytes's check (types.rs:337-349)
        s.load_state_dict(p)
    with_section(offset=len(head) + 1)
    with pytest.raises(s.SerializeError, match="section at"):
        s.load_state_dict(p)
    with_section(extra=b"\0")
    with pytest.raises(s.SerializeError, match="trailing"):
        s.load_state_dict(p)
    with pytest.raises(s.SerializeError):
        s.load_state_dict(tmp_path / "missing.axonml")
    with pytest.raises(s.SerializeError, match="safetensors"):
        s.save_state_dict(_example(), tmp_path / "m.safetensors")
    pj = tmp_path / "m.json"
    pj.write_text('{"entries": {"w": {"data": {"shape": [1], "values": [null]}, "requires_grad": true}}}')
    with pytest.raises(s.SerializeError, match="null"):
        s.load_state_dict(pj)
    pj.write_text("{")
    with pytest.raises(s.SerializeError):
        s.load_state_dict(pj)
    with pytest.raises(s.SerializeError, match="does not hold"):
        s.TensorData([2, 2], [1.0]).to_tensor()


@pytest.mark.gpu
def test_quantized_model_survives_save_and_load(ctx, tmp_path):
    from tests.util import MATMUL_RTOL, REL_FLOOR, max_rel_err

    rng = np.random.default_rng(3)
    sd = s.StateDict()
    sd.insert("fc.weight", s.TensorData.from_tensor(rng.standard_normal((96, 512)).astype(np.float32) * 0.05))
    sd.insert("fc.bias", s.TensorData.from_tensor(rng.standard_normal(96).astype(np.float32)))
    qsd = s.quantize_state_dict(sd, q.QuantType.Q4_K, ctx)
    assert list(qsd.keys()) == ["fc.bias"] and list(qsd.quantized) == ["fc.weight"]
    want_blocks = o.quantize(o.Q4_K, sd.get("fc.weight").data.to_tensor())
    assert np.array_equal(qsd.get_quantized("fc.weight").data, want_blocks)  # the device quantiser, bit for bit
    for ext in ("axonml", "json"):
        p = tmp_path / f"m.{ext}"
        s.save_state_dict(qsd, p)
        back = s.load_state_dict(p)
        lin = q.QuantizedLinear(back.get_quantized("fc.weight"), back.get("fc.bias").data.to_tensor(), ctx)
        x = rng.standard_normal((3, 512)).astype(np.float32)
        ref = x.astype(np.float64) @ o.dequantize(o.Q4_K, want_blocks, 96 * 512).reshape(96, 512).astype(np.float64).T
        ref += sd.get("fc.bias").data.values
        assert max_rel_err(lin.forward(x), ref, REL_FLOOR) <= MATMUL_RTOL
    assert p.stat().st_size > 0 and (tmp_path / "m.axonml").stat().st_size < 96 * 512 * 4 / 6  # 4.5 bits per weight on disk
