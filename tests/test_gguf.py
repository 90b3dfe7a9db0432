"""GGUF interop: the oracle's block conversion pinned against ggml's own element formulas, the container
reader against a file assembled by hand in this test, and (GPU) the device conversion, the writer and the
LLaMA loader.  Conversion is byte work: the bar is bit-exact.

Parity note: the reference has no GGUF code (only the extension string, cli/src/commands/quant.rs:218), so
the block layouts are anchored on the GGUF / ggml specification; what pins the conversion to the
reference is that the converted image, run through the reference's dequantiser (already pinned by the
reference's own vectors), reproduces ggml's values exactly."""
import struct

import numpy as np
import pytest

import oracle as o
from axonml_amd import gguf
from axonml_amd import quant as q


# ---------------------------------------------------------------------------
# oracle pins (CPU)
# ---------------------------------------------------------------------------
def _ggml_block_q4_0(d_bits, elems):
    """A ggml block_q4_0 written from the spec: f16 d, then qs[j] = (elems[j] + 8) | (elems[j + 16] + 8) << 4."""
    qs = bytes(((elems[j] + 8) & 0xF) | (((elems[j + 16] + 8) & 0xF) << 4) for j in range(16))
    return struct.pack("<H", d_bits) + qs


def test_known_answer_q4_0_block():
    # elements -8..7 twice over; scale 0.5 (f16 0x3800)
    elems = [(i % 16) - 8 for i in range(32)]
    g = np.frombuffer(_ggml_block_q4_0(0x3800, elems), dtype=np.uint8)
    # ggml order: byte j holds elements j and j + 16, which are equal here
    assert list(g[2:]) == [j | (j << 4) for j in range(16)]
    n = o.gguf_convert(o.Q4_0, g, to_gguf=False)
    # reference order (types.rs:190-198): byte i holds elements 2i and 2i + 1
    want = [((2 * i) % 16) | (((2 * i + 1) % 16) << 4) for i in range(16)]
    assert list(n[:2]) == [0x00, 0x38] and list(n[2:]) == want
    # ... and the reference's dequantiser (dequantize.rs:116-121) gives ggml's values
    assert np.array_equal(o.dequantize(o.Q4_0, n, 32), np.array(elems, dtype=np.float32) * 0.5)


def test_one_hot_nibbles_land_where_the_spec_says():
    for e in range(32):
        g = np.zeros(18, dtype=np.uint8)
        g[0:2] = [0x00, 0x3C]  # d = 1.0
        g[2:] = 0x88           # every element 0
        j, hi = e % 16, e // 16
        g[2 + j] = (0x8F if not hi else 0xF8)  # element e = 15 - 8 = 7
        n = o.gguf_convert(o.Q4_0, g, to_gguf=False)
        vals = o.dequantize(o.Q4_0, n, 32)
        assert vals[e] == 7.0 and np.count_nonzero(vals) == 1, e
        assert n[2 + e // 2] == (0x8F if e % 2 == 0 else 0xF8)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1])
def test_converted_blocks_dequantise_to_ggml_values(qtype):
    rng = np.random.default_rng(3 + qtype)
    bb = 18 if qtype == o.Q4_0 else 20
    g = rng.integers(0, 256, size=500 * bb, dtype=np.uint8).reshape(500, bb)
    g[:, 1] &= 0x3F  # keep the f16 scales (and mins) finite and modest
    if qtype == o.Q4_1:
        g[:, 3] &= 0x3F
    g = g.reshape(-1)
    n = o.gguf_convert(qtype, g, to_gguf=False)
    assert np.array_equal(o.dequantize(qtype, n, 500 * 32), o.ggml_dequantize(qtype, g))
    assert np.array_equal(o.gguf_convert(qtype, n, to_gguf=True), g)  # and back


def test_ggml_formula_against_numpy():
    # ggml's dequantize_row_q4_1, restated once more in numpy: y[j] = d * (qs[j] & 15) + m, y[j + 16] = d * (qs[j] >> 4) + m
    rng = np.random.default_rng(9)
    g = rng.integers(0, 256, size=40 * 20, dtype=np.uint8).reshape(40, 20)
    g[:, 1] &= 0x3F
    g[:, 3] &= 0x3F
    d = g[:, 0:2].copy().view(np.float16).astype(np.float32)
    m = g[:, 2:4].copy().view(np.float16).astype(np.float32)
    qs = g[:, 4:]
    want = np.concatenate([(qs & 15).astype(np.float32) * d + m, (qs >> 4).astype(np.float32) * d + m], axis=1)
    assert np.array_equal(o.ggml_dequantize(o.Q4_1, g.reshape(-1)).reshape(40, 32), want)


@pytest.mark.parametrize("qtype", [o.Q8_0, o.Q5_0, o.Q5_1, o.Q4_K, o.Q5_K, o.Q6_K, o.F16, o.F32])
def test_other_types_are_byte_identical(qtype):
    rng = np.random.default_rng(qtype)
    n = 512
    b = rng.integers(0, 256, size=o.packed_bytes(qtype, n), dtype=np.uint8)
    assert np.array_equal(o.gguf_convert(qtype, b, to_gguf=False), b)


# ---------------------------------------------------------------------------
# container reader against a hand-assembled file (CPU; loads the C library for the type table only)
# ---------------------------------------------------------------------------
def _s(x):
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _hand_made_file(tmp_path, alignment=None, version=3, tensor_type=2, bad_offset=False, truncate=0):
    kv = [_s("general.architecture") + struct.pack("<I", 8) + _s("llama"),
          _s("llama.block_count") + struct.pack("<II", 4, 2),
          _s("llama.rope.freq_base") + struct.pack("<If", 6, 10000.0),
          _s("some.flag") + struct.pack("<I?", 7, True),
          _s("some.i64") + struct.pack("<Iq", 11, -5),
          _s("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, 3) + _s("a") + _s("bc") + _s("def"),
          _s("some.floats") + struct.pack("<IIQ", 9, 6, 2) + struct.pack("<ff", 1.5, -2.0)]
    if alignment:
        kv.append(_s("general.alignment") + struct.pack("<II", 4, alignment))
    al = alignment or 32
    t0 = np.arange(2 * 64, dtype=np.uint8)[: 2 * 2 * 18]  # [2, 64] Q4_0 = 4 blocks of 18 bytes
    t1 = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    off1 = (t0.size + al - 1) // al * al
    if bad_offset:
        off1 += 1
    infos = [_s("blk.0.w") + struct.pack("<I", 2) + struct.pack("<QQ", 64, 2) + struct.pack("<IQ", tensor_type, 0),
             _s("norm") + struct.pack("<I", 1) + struct.pack("<Q", 3) + struct.pack("<IQ", 0, off1)]
    head = b"GGUF" + struct.pack("<IQQ", version, len(infos), len(kv)) + b"".join(kv) + b"".join(infos)
    body = head + b"\0" * (-len(head) % al) + t0.tobytes() + b"\0" * (off1 - t0.size) + t1.tobytes()
    if truncate:
        body = body[:-truncate]
    p = tmp_path / "hand.gguf"
    p.write_bytes(body)
    return str(p), t0, t1


def test_tokenizer_from_the_files_metadata(tmp_path):
    # the reference's BPE over a GGUF vocabulary: "low" + "er" by the merge list, ids as the array orders them
    tokens = ["<unk>", "<s>", "</s>", "l", "o", "w", "e", "r", " ", "lo", "low", "er", "lower"]
    md = {"general.architecture": "llama", "tokenizer.ggml.model": "gpt2", "tokenizer.ggml.tokens": tokens,
          "tokenizer.ggml.merges": ["l o", "lo w", "e r", "low er"], "tokenizer.ggml.bos_token_id": 1,
          "tokenizer.ggml.eos_token_id": 2, "tokenizer.ggml.unknown_token_id": 0}
    path = str(tmp_path / "tok.gguf")
    gguf.write_gguf(path, md, {"norm": np.ones(4, np.float32)})
    with gguf.GGUFReader(path) as r:
        tok = gguf.tokenizer_from_metadata(r.metadata)
    assert tok.vocab_size() == len(tokens) and tok.bos_token_id() == 1 and tok.eos_token_id() == 2
    assert tok.encode("lower") == [1, 12] and tok.encode("low") == [1, 10]  # encode() puts the BOS token in front
    assert tok.encode_with_options("lower", False, True) == [12, 2]
    assert tok.decode([10, 11]) == "lower"
    assert tok.encode_with_options("z", False, False) == [0]  # no such piece: the unknown token
    with pytest.raises(gguf.GGUFError):
        gguf.tokenizer_from_metadata({"general.architecture": "llama"})


def test_bf16_tensors_widen_exactly(tmp_path):
    # ggml type 30: the bit pattern is the upper half of the f32 word (1.0 = 0x3F80, -2.5 = 0xC020, the largest finite
    # value 0x7F7F, a subnormal 0x0001); such a tensor reads as f32, and as a linear it is carried as an F32 weight
    bits = np.array([[0x3F80, 0xC020, 0x7F7F, 0x0001], [0x0000, 0x8000, 0x3DCD, 0x4049]], np.uint16)
    path = str(tmp_path / "bf16.gguf")
    gguf.write_gguf(path, {"general.architecture": "llama"}, {"w": ("BF16", bits)})
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    assert want[0, 0] == 1.0 and want[0, 1] == -2.5
    with gguf.GGUFReader(path) as r:
        assert r.info("w").ggml_type == 30 and r.info("w").shape == (2, 4) and r.info("w").nbytes == 16
        got = gguf.load_f32(r, "w")
        assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
        qt = gguf.load_quantized_tensor(r, "w")
        assert qt.quant_type == q.QuantType.F32 and qt.shape == [2, 4]
        assert np.array_equal(qt.data.view(np.float32).view(np.uint32), want.reshape(-1).view(np.uint32))


@pytest.mark.parametrize("alignment", [None, 64])
def test_reader_parses_a_hand_assembled_file(tmp_path, alignment):
    path, t0, t1 = _hand_made_file(tmp_path, alignment)
    with gguf.GGUFReader(path) as r:
        assert r.version == 3 and r.alignment == (alignment or 32)
        md = r.metadata
        assert md["general.architecture"] == "llama" and md["llama.block_count"] == 2 and md["some.flag"] is True
        assert md["some.i64"] == -5 and md["llama.rope.freq_base"] == 10000.0
        assert md["tokenizer.ggml.tokens"] == ["a", "bc", "def"]
        assert md["some.floats"].dtype == np.float32 and list(md["some.floats"]) == [1.5, -2.0]
        w = r.info("blk.0.w")
        assert w.shape == (2, 64) and w.quant_type == q.QuantType.Q4_0 and w.nbytes == 72  # ne = [64, 2] reversed
        assert np.array_equal(r.tensor_bytes("blk.0.w"), t0)
        assert np.array_equal(gguf.load_f32(r, "norm"), t1)
        with pytest.raises(gguf.GGUFError, match="no tensor"):
            r.info("nope")


def test_reader_errors(tmp_path):
    p = tmp_path / "x.gguf"
    p.write_bytes(b"GGML" + b"\0" * 40)
    with pytest.raises(gguf.GGUFError, match="magic"):
        gguf.GGUFReader(str(p))
    p.write_bytes(b"GGUF")
    with pytest.raises(gguf.GGUFError, match="truncated"):
        gguf.GGUFReader(str(p))
    with pytest.raises(gguf.GGUFError, match="version"):
        gguf.GGUFReader(_hand_made_file(tmp_path, version=1)[0])
    with pytest.raises(gguf.GGUFError, match="big-endian"):
        gguf.GGUFReader(_hand_made_file(tmp_path, version=0x03000000)[0])
    with pytest.raises(gguf.GGUFError, match="aligned"):
        gguf.GGUFReader(_hand_made_file(tmp_path, bad_offset=True)[0])
    with pytest.raises(gguf.GGUFError, match="past the end"):
        gguf.GGUFReader(_hand_made_file(tmp_path, truncate=8)[0])
    with pytest.raises(gguf.GGUFError, match="power of two"):
        gguf.GGUFReader(_hand_made_file(tmp_path, alignment=24)[0])
    # a ggml type without a kernel here (Q3_K = 11) parses, and is refused when its data is asked for
    with gguf.GGUFReader(_hand_made_file(tmp_path, tensor_type=11)[0]) as r:
        assert r.info("blk.0.w").quant_type is None
        with pytest.raises(gguf.GGUFError, match="Q3_K"):
            r.tensor_bytes("blk.0.w")
    assert issubclass(gguf.GGUFError, q.QuantError)


def test_rope_row_permutation_is_the_inverse_of_the_converters():
    # llama.cpp's converter: w.reshape(n_head, 2, d/2, k).swapaxes(1, 2).reshape(w.shape)
    n_head, d, k = 3, 8, 5
    w = np.arange(n_head * d * k).reshape(n_head * d, k)
    file_rows = w.reshape(n_head, 2, d // 2, k).swapaxes(1, 2).reshape(w.shape)
    assert np.array_equal(file_rows[gguf.rope_rows_to_half_split(n_head * d, n_head)], w)


# ---------------------------------------------------------------------------
# device conversion, writer, loader (GPU)
# ---------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1])
@pytest.mark.parametrize("nblocks", [1, 7, 255, 256, 257, 1000, 40000])
def test_device_conversion_is_bit_exact_both_ways(ctx, qtype, nblocks):
    rng = np.random.default_rng(nblocks + qtype)
    bb = o.lib().axo_bytes_per_block(qtype)
    g = rng.integers(0, 256, size=nblocks * bb, dtype=np.uint8)
    n = gguf.convert_blocks(qtype, g, False, ctx)
    assert np.array_equal(n, o.gguf_convert(qtype, g, to_gguf=False))
    assert np.array_equal(gguf.convert_blocks(qtype, n, True, ctx), g)


@pytest.mark.gpu
def test_device_conversion_on_device_buffers_in_place(ctx):
    from axonml_amd._lib import MEM_DEVICE

    rng = np.random.default_rng(5)
    g = rng.integers(0, 256, size=3000 * 18, dtype=np.uint8)
    d = ctx.to_device(g)
    ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, o.Q4_0, d, d, 3000, 0, MEM_DEVICE))
    assert np.array_equal(ctx.to_host(d, g.size, np.uint8), o.gguf_convert(o.Q4_0, g, to_gguf=False))
    ctx.free(d)
    # identical types are a copy; unknown types and directions are refused
    b = rng.integers(0, 256, size=34 * 5, dtype=np.uint8)
    assert np.array_equal(gguf.convert_blocks(o.Q8_0, b, False, ctx), b)
    with pytest.raises(q.QuantError):
        ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, 99, b.ctypes.data, b.ctypes.data, 1, 0, 0))
    with pytest.raises(q.QuantError):
        ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, o.Q4_0, b.ctypes.data, b.ctypes.data, 1, 7, 0))


@pytest.mark.gpu
def test_write_then_read_round_trip_and_matmul_on_ggml_values(ctx, tmp_path):
    rng = np.random.default_rng(12)
    n, k = 48, 512
    tensors, packed = {}, {}
    for qtype in (o.Q4_0, o.Q4_1, o.Q5_1, o.Q8_0, o.Q4_K, o.Q5_K, o.Q6_K):
        packed[qtype] = o.quantize(qtype, (rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        tensors[f"w.{o.TYPE_NAMES[qtype]}"] = q.QuantizedTensor([n, k], qtype, packed[qtype])
    tensors["norm"] = rng.standard_normal(k).astype(np.float32)
    tensors["half"] = rng.standard_normal((3, 32)).astype(np.float16)
    path = str(tmp_path / "t.gguf")
    gguf.write_gguf(path, {"general.architecture": "llama", "x.count": 5, "x.name": "abc", "x.eps": 1e-5}, tensors, ctx)
    x = rng.standard_normal((1, k)).astype(np.float32)
    with gguf.GGUFReader(path) as r:
        assert r.metadata["x.count"] == 5 and r.metadata["x.name"] == "abc" and abs(r.metadata["x.eps"] - 1e-5) < 1e-12
        for qtype in packed:
            name = f"w.{o.TYPE_NAMES[qtype]}"
            # the file holds ggml-order images ...
            want_file = o.gguf_convert(qtype, packed[qtype], to_gguf=True)
            assert np.array_equal(r.tensor_bytes(name), want_file)
            # ... which load back to the reference-order bytes
            qt = gguf.load_quantized_tensor(r, name, ctx)
            assert qt.shape == [n, k] and np.array_equal(qt.data, packed[qtype])
            # and multiply like ggml's values: for Q4_0 / Q4_1 against ggml's own dequantiser on the file bytes
            wd = (o.ggml_dequantize(qtype, want_file) if qtype in (o.Q4_0, o.Q4_1) else o.dequantize(qtype, packed[qtype], n * k))
            y = q.quantized_matmul(x, qt, None, ctx)
            ref = o.matmul_f64(wd.reshape(n, k), x)
            assert np.abs(y - ref).max() <= 1e-3 * np.abs(ref).max()  # tolerance of the quantized matmul, normwise
        assert np.array_equal(gguf.load_f32(r, "norm", ctx), tensors["norm"])
        assert np.array_equal(gguf.load_f32(r, "half", ctx), tensors["half"].astype(np.float32))
        assert np.array_equal(gguf.load_f32(r, "w.Q4_0", ctx).reshape(-1), o.dequantize(o.Q4_0, packed[o.Q4_0], n * k))


def _q4_k_m_like(c, w, seed, ffn_too=False):
    """The weights of a Q4_K model with the linears llama.cpp's Q4_K_M recipe keeps at six bits requantised to Q6_K:
    attn_v and ffn_down of every other layer, and the output matrix (ffn_too: ffn_up of those layers as well, which
    no stock recipe does: a gate/up pair of two types).  Returns name -> type for what changed."""
    from tests.decode_common import LIN_SHAPES

    rng = np.random.default_rng(seed)
    types = {}
    for i, L in enumerate(w["layers"]):
        if i % 2 == 0:
            for name in ("v", "down", "up") if ffn_too else ("v", "down"):
                n, k = LIN_SHAPES(c)[name]
                L[name] = o.quantize(o.Q6_K, (rng.standard_normal((n, k)) * 0.06).astype(np.float32))
                types[(i, name)] = o.Q6_K
    w["head"] = o.quantize(o.Q6_K, (rng.standard_normal((c["vocab_size"], c["hidden_size"])) * 0.06).astype(np.float32))
    types[(-1, "head")] = o.Q6_K
    return types


@pytest.mark.gpu
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_K, o.Q5_K, o.Q6_K, "Q4_K_M", "Q4_K_M+up"])
def test_llama_loaded_from_gguf_decodes_like_the_oracle(ctx, tmp_path, qtype):
    from tests.decode_common import LIN_SHAPES, load_oracle, random_weights, tiny_config
    from tests.util import DECODE_FLOOR, DECODE_RTOL, max_rel_err

    c = tiny_config()
    mixed = {}
    if qtype in ("Q4_K_M", "Q4_K_M+up"):
        ffn_too = qtype.endswith("+up")
        qtype = o.Q4_K
        w = random_weights(c, 77, qtype=qtype)
        mixed = _q4_k_m_like(c, w, 78, ffn_too)
    else:
        w = random_weights(c, 77, qtype=qtype)
    w["types"] = mixed
    cpu = load_oracle(c, w)
    # the file as llama.cpp's converter lays it out: q/k rows permuted per head, llama.* metadata, blk.N.* names
    md = {"general.architecture": "llama", "llama.block_count": c["num_layers"], "llama.embedding_length": c["hidden_size"],
          "llama.feed_forward_length": c["intermediate_size"], "llama.attention.head_count": c["num_heads"],
          "llama.attention.head_count_kv": c["num_kv_heads"], "llama.context_length": c["max_seq_len"],
          "llama.attention.layer_norm_rms_epsilon": c["rms_norm_eps"], "llama.rope.freq_base": c["rope_theta"]}
    tensors = {"token_embd.weight": w["emb"].view(np.float16).reshape(c["vocab_size"], c["hidden_size"]),
               "output_norm.weight": w["final_norm"]}

    def converter_order(packed, n_rows, heads):
        rows = np.asarray(packed).reshape(n_rows, -1)
        d = n_rows // heads
        return rows.reshape(heads, 2, d // 2, -1).swapaxes(1, 2).reshape(n_rows, -1)

    stems = {"q": "attn_q", "k": "attn_k", "v": "attn_v", "o": "attn_output", "gate": "ffn_gate", "up": "ffn_up", "down": "ffn_down"}
    for i, L in enumerate(w["layers"]):
        tensors[f"blk.{i}.attn_norm.weight"], tensors[f"blk.{i}.ffn_norm.weight"] = L["norm0"], L["norm1"]
        for name, (n, k) in LIN_SHAPES(c).items():
            data = L[name]
            if name in ("q", "k"):
                data = converter_order(data, n, c["num_heads"] if name == "q" else c["num_kv_heads"])
            tensors[f"blk.{i}.{stems[name]}.weight"] = q.QuantizedTensor([n, k], mixed.get((i, name), qtype), data)
    tensors["output.weight"] = q.QuantizedTensor([c["vocab_size"], c["hidden_size"]], mixed.get((-1, "head"), qtype), w["head"])
    path = str(tmp_path / "tiny-llama.gguf")
    gguf.write_gguf(path, md, tensors, ctx)

    gpu = gguf.load_llama(path, ctx)
    assert gpu.cfg.vocab_size == c["vocab_size"] and gpu.cfg.num_key_value_heads == c["num_kv_heads"]
    tok = 5
    for pos in range(12):
        c_next, c_logits = cpu.forward(tok, pos)
        g_next, g_logits = gpu.forward(tok)
        assert max_rel_err(g_logits, c_logits, DECODE_FLOOR) <= DECODE_RTOL, pos
        assert g_next == c_next, pos
        tok = c_next
    gpu.close()
    cpu.close()
