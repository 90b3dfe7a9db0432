"""GGUF container: reader, writer and a LLaMA/Mistral loader for the decode path.

The reference accepts ``.gguf`` as a file extension (crates/axonml-cli/src/commands/quant.rs:218) and
stops there; its `axonml quant convert` writes nothing a reader could load (quant.rs:171-180).  This module
implements the GGUF v2/v3 container as specified by ggml: little-endian header, typed metadata, tensor
table, aligned data section.  Tensor payloads are ggml block images; `axq_gguf_convert_blocks` (device)
turns Q4_0 / Q4_1 images into the reference's nibble order and back, every other supported type is
byte-identical (Q5_K and Q6_K among them: the reference has no such types, the blocks are ggml's).  ggml types this library
has no kernel for (Q2_K, Q3_K, IQ*, ...) raise GGUFError.

Tensor names and metadata keys of the loader follow llama.cpp's converter for the `llama` architecture,
mapped onto the reference's LLaMA module names (crates/axonml-llm/src/llama.rs:782-822).
"""
import mmap
import os
import struct

import numpy as np

from . import _lib
from ._lib import MEM_HOST
from .quant import QuantError, QuantizedTensor, QuantType, default_context

GGUF_MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# metadata value types
T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_SCALAR = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<?",
           T_U64: "<Q", T_I64: "<q", T_F64: "<d"}
_NP = {T_U8: "<u1", T_I8: "<i1", T_U16: "<u2", T_I16: "<i2", T_U32: "<u4", T_I32: "<i4", T_F32: "<f4", T_BOOL: "?",
       T_U64: "<u8", T_I64: "<i8", T_F64: "<f8"}

# ggml_type numbers (names for messages; block geometry for the ones this library can hold)
GGML_TYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K",
                   11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 30: "BF16"}


GGML_BF16 = 30


class GGUFError(QuantError):
    pass


def _axq_type(ggml_type):
    t = _lib.load_library().axq_type_from_ggml(int(ggml_type))
    return None if t < 0 else QuantType(t)


class GGUFTensorInfo:
    """One row of the tensor table.  `shape` is row-major (outermost first), i.e. ggml's `ne` reversed."""

    def __init__(self, name, shape, ggml_type, offset):
        self.name, self.shape, self.ggml_type, self.offset = name, tuple(int(s) for s in shape), int(ggml_type), int(offset)
        self.quant_type = _axq_type(ggml_type)
        self.numel = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = None
        if self.quant_type is not None:
            bs = self.quant_type.block_size()
            inner = self.shape[-1] if self.shape else 1
            if inner % bs:
                raise GGUFError(f"tensor {name}: innermost dimension {inner} is not a multiple of the {self.quant_type} block size {bs}")
            self.nbytes = self.numel // bs * self.quant_type.bytes_per_block()
        elif self.ggml_type == GGML_BF16:  # no block type of its own here: widened to f32 (exactly) when it is read
            self.nbytes = self.numel * 2

    def __repr__(self):
        return f"GGUFTensorInfo({self.name!r}, shape={self.shape}, ggml_type={GGML_TYPE_NAMES.get(self.ggml_type, self.ggml_type)})"


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, n):
        if n < 0 or self.pos + n > len(self.buf):
            raise GGUFError("truncated GGUF file")
        v = self.buf[self.pos:self.pos + n]
        self.pos += n
        return v

    def scalar(self, fmt):
        return struct.unpack(fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self):
        n = self.scalar("<Q")
        try:
            return bytes(self.take(n)).decode("utf-8")
        except UnicodeDecodeError as e:
            raise GGUFError(f"metadata string is not UTF-8: {e}") from None

    def value(self, vtype, depth=0):
        if vtype in _SCALAR:
            return self.scalar(_SCALAR[vtype])
        if vtype == T_STR:
            return self.string()
        if vtype == T_ARR:
            if depth > 4:
                raise GGUFError("metadata arrays nested too deeply")
            etype, count = self.scalar("<I"), self.scalar("<Q")
            if etype in _NP:
                dt = np.dtype(_NP[etype])
                return np.frombuffer(self.take(count * dt.itemsize), dtype=dt).copy()
            return [self.value(etype, depth + 1) for _ in range(count)]
        raise GGUFError(f"unknown metadata value type {vtype}")


class GGUFReader:
    """Memory-maps a GGUF file; `metadata` is a dict, `tensors` a dict name -> GGUFTensorInfo."""

    def __init__(self, path):
        self.path = path
        self._f = open(path, "rb")
        try:
            size = os.fstat(self._f.fileno()).st_size
            if size < 24:
                raise GGUFError("truncated GGUF file")
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        except Exception:
            self._f.close()
            raise
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    def _parse(self):
        view = memoryview(self._mm)
        try:
            self._parse_header(_Cursor(view))
        finally:
            view.release()

    def _parse_header(self, c):
        if bytes(c.take(4)) != GGUF_MAGIC:
            raise GGUFError("not a GGUF file (bad magic)")
        self.version = c.scalar("<I")
        if self.version not in (2, 3):
            if self.version in (0x02000000, 0x03000000):
                raise GGUFError("big-endian GGUF files are not supported")
            raise GGUFError(f"unsupported GGUF version {self.version}")
        n_tensors, n_kv = c.scalar("<Q"), c.scalar("<Q")
        self.metadata = {}
        for _ in range(n_kv):
            key = c.string()
            self.metadata[key] = c.value(c.scalar("<I"))
        self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"general.alignment {self.alignment} is not a power of two")
        self.tensors = {}
        for _ in range(n_tensors):
            name = c.string()
            nd = c.scalar("<I")
            if nd > 4:
                raise GGUFError(f"tensor {name}: {nd} dimensions")
            ne = [c.scalar("<Q") for _ in range(nd)]
            ggml_type, offset = c.scalar("<I"), c.scalar("<Q")
            if name in self.tensors:
                raise GGUFError(f"duplicate tensor name {name}")
            self.tensors[name] = GGUFTensorInfo(name, ne[::-1], ggml_type, offset)
        self.data_start = (c.pos + self.alignment - 1) // self.alignment * self.alignment
        for t in self.tensors.values():
            if t.offset % self.alignment:
                raise GGUFError(f"tensor {t.name}: offset {t.offset} is not aligned to {self.alignment}")
            if t.nbytes is not None and self.data_start + t.offset + t.nbytes > len(self._mm):
                raise GGUFError(f"tensor {t.name}: data runs past the end of the file")

    def info(self, name):
        try:
            return self.tensors[name]
        except KeyError:
            raise GGUFError(f"no tensor named {name}") from None

    def tensor_bytes(self, name):
        """The tensor's ggml block images as a uint8 view of the mapped file."""
        t = self.info(name)
        if t.quant_type is None and t.ggml_type != GGML_BF16:
            raise GGUFError(f"tensor {name}: ggml type {GGML_TYPE_NAMES.get(t.ggml_type, t.ggml_type)} is not supported "
                            f"(supported: F32, F16, BF16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K)")
        return np.frombuffer(self._mm, dtype=np.uint8, count=t.nbytes, offset=self.data_start + t.offset)

    def close(self):
        mm, self._mm = getattr(self, "_mm", None), None
        if mm is not None:
            try:
                mm.close()
            except BufferError:
                pass  # a caller still holds a view; the map goes with it
        f, self._f = getattr(self, "_f", None), None
        if f is not None:
            f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def convert_blocks(quant_type, blocks, to_gguf, ctx=None):
    """ggml-order block images <-> reference-order images (device kernel; identical types are copied)."""
    ctx = ctx or default_context()
    src = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    bb = QuantType(quant_type).bytes_per_block()
    if src.size % bb:
        raise GGUFError(f"{src.size} bytes are not whole {QuantType(quant_type)} blocks of {bb}")
    out = np.empty_like(src)
    ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, int(quant_type), src.ctypes.data, out.ctypes.data, src.size // bb,
                                              1 if to_gguf else 0, MEM_HOST))
    return out


def load_quantized_tensor(reader, name, ctx=None):
    """GGUF tensor -> QuantizedTensor in the reference's block order (shape row-major)."""
    t = reader.info(name)
    raw = reader.tensor_bytes(name)
    if t.ggml_type == GGML_BF16:  # as f32, which holds every bf16 value
        return QuantizedTensor(list(t.shape), QuantType.F32, _bf16_to_f32(raw).view(np.uint8).reshape(-1))
    return QuantizedTensor(list(t.shape), t.quant_type, convert_blocks(t.quant_type, raw, False, ctx))


def _bf16_to_f32(raw):
    """bf16 bit patterns (little-endian bytes) -> float32: the pattern is the upper half of the f32 word."""
    return (raw.view("<u2").astype(np.uint32) << 16).view(np.float32)


def load_f32(reader, name, ctx=None):
    """GGUF tensor of any supported type as float32 (dequantised on the device when it is quantised)."""
    from .quant import dequantize_tensor

    t = reader.info(name)
    raw = reader.tensor_bytes(name)
    if t.quant_type == QuantType.F32:
        return raw.view("<f4").reshape(t.shape).copy()
    if t.quant_type == QuantType.F16:
        return raw.view("<f2").astype(np.float32).reshape(t.shape)
    if t.ggml_type == GGML_BF16:
        return _bf16_to_f32(raw).reshape(t.shape)
    return np.asarray(dequantize_tensor(load_quantized_tensor(reader, name, ctx), ctx)).reshape(t.shape)


# ---------------------------------------------------------------------------
# writer
# ---------------------------------------------------------------------------
def _enc_string(s):
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _enc_value(v):
    if isinstance(v, bool):
        return struct.pack("<I?", T_BOOL, v)
    if isinstance(v, (int, np.integer)):
        v = int(v)
        if 0 <= v < 2 ** 32:
            return struct.pack("<II", T_U32, v)
        return struct.pack("<Iq", T_I64, v) if v < 0 else struct.pack("<IQ", T_U64, v)
    if isinstance(v, (float, np.floating)):
        return struct.pack("<If", T_F32, float(v))
    if isinstance(v, str):
        return struct.pack("<I", T_STR) + _enc_string(v)
    if isinstance(v, np.ndarray):
        for code, dt in _NP.items():
            if v.dtype == np.dtype(dt):
                return struct.pack("<IIQ", T_ARR, code, v.size) + np.ascontiguousarray(v).tobytes()
        raise GGUFError(f"metadata array of dtype {v.dtype}")
    if isinstance(v, (list, tuple)) and all(isinstance(x, str) for x in v):
        return struct.pack("<IIQ", T_ARR, T_STR, len(v)) + b"".join(_enc_string(x) for x in v)
    raise GGUFError(f"cannot encode metadata value {v!r}")


def write_gguf(path, metadata, tensors, ctx=None, alignment=DEFAULT_ALIGNMENT):
    """Writes a GGUF v3 file.  `tensors`: name -> QuantizedTensor (reference block order; converted to ggml
    order on the device), a float32 / float16 numpy array, or ("BF16", uint16 array of bf16 bit patterns)."""
    lib = _lib.load_library()
    metadata = dict(metadata)
    if alignment != DEFAULT_ALIGNMENT:
        metadata["general.alignment"] = int(alignment)
    payloads, infos, offset = [], [], 0
    for name, t in tensors.items():
        if isinstance(t, QuantizedTensor):
            ggml_type = lib.axq_type_to_ggml(int(t.quant_type))
            data = convert_blocks(t.quant_type, t.data, True, ctx)
            shape = t.shape
        elif isinstance(t, tuple) and len(t) == 2 and t[0] == "BF16":
            a = np.ascontiguousarray(t[1], dtype=np.uint16)
            ggml_type, data, shape = GGML_BF16, a.view(np.uint8).reshape(-1), a.shape
        else:
            a = np.ascontiguousarray(t)
            if a.dtype not in (np.float32, np.float16):
                raise GGUFError(f"tensor {name}: dtype {a.dtype}")
            ggml_type = 0 if a.dtype == np.float32 else 1
            data, shape = a.view(np.uint8).reshape(-1), a.shape
        infos.append(_enc_string(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape[::-1])
                     + struct.pack("<IQ", ggml_type, offset))
        payloads.append(data)
        offset = (offset + data.size + alignment - 1) // alignment * alignment
    head = GGUF_MAGIC + struct.pack("<IQQ", 3, len(payloads), len(metadata))
    head += b"".join(_enc_string(k) + _enc_value(v) for k, v in metadata.items()) + b"".join(infos)
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-len(head) % alignment))
        for data in payloads:
            f.write(data.tobytes())
            f.write(b"\0" * (-data.size % alignment))


# ---------------------------------------------------------------------------
# LLaMA / Mistral loader
# ---------------------------------------------------------------------------
_LINEAR_NAMES = {"q": "attn_q", "k": "attn_k", "v": "attn_v", "o": "attn_output", "gate": "ffn_gate", "up": "ffn_up",
                 "down": "ffn_down"}


def rope_rows_to_half_split(n_rows, n_heads):
    """Row order that undoes llama.cpp's permutation of q/k projection rows.

    Its converter reorders the rows of every head so that ggml's RoPE can rotate adjacent pairs; the
    reference rotates element i with element i + head_dim / 2 (RotaryEmbedding, llama.rs:223-252).  Within a
    head of d rows, file row 2i + t holds the row that the half-split convention calls t * d/2 + i.
    Returns `perm` with native_rows = file_rows[perm]."""
    d = n_rows // n_heads
    i = np.arange(d // 2)
    within = np.concatenate([2 * i, 2 * i + 1])  # native row t*d/2 + i  <-  file row 2i + t
    return (np.arange(n_heads)[:, None] * d + within[None, :]).reshape(-1)


def llama_config_from_metadata(md, max_position_embeddings=None):
    arch = md.get("general.architecture", "llama")
    if arch != "llama":
        raise GGUFError(f"architecture {arch!r}: only `llama` (LLaMA / Mistral) is handled")

    def need(key):
        if key not in md:
            raise GGUFError(f"metadata key {key} is missing")
        return md[key]

    hidden, heads = int(need("llama.embedding_length")), int(need("llama.attention.head_count"))
    ctx_len = int(md.get("llama.context_length", 4096))
    return dict(hidden_size=hidden, intermediate_size=int(need("llama.feed_forward_length")),
                num_hidden_layers=int(need("llama.block_count")), num_attention_heads=heads,
                num_key_value_heads=int(md.get("llama.attention.head_count_kv", heads)),
                head_dim=int(md.get("llama.attention.key_length", hidden // heads)),
                max_position_embeddings=int(max_position_embeddings or min(ctx_len, 4096)),
                rms_norm_eps=float(md.get("llama.attention.layer_norm_rms_epsilon", 1e-5)),
                rope_theta=float(md.get("llama.rope.freq_base", 10000.0)),
                sliding_window=int(md.get("llama.attention.sliding_window", 0)))


def load_llama(path, ctx=None, max_position_embeddings=None, permuted_qk=True):
    """GGUF file of the `llama` architecture -> QuantizedLlama with every linear device-resident.

    `permuted_qk`: the file's q/k rows are in llama.cpp's converter order (true for files it produced)."""
    from .decode import QuantizedLlama

    ctx = ctx or default_context()
    with GGUFReader(path) as r:
        cfg = llama_config_from_metadata(r.metadata, max_position_embeddings)
        emb_info = r.info("token_embd.weight")
        cfg["vocab_size"] = int(r.metadata.get("llama.vocab_size", emb_info.shape[0]))
        model = QuantizedLlama(ctx, **cfg)
        emb = load_f32(r, "token_embd.weight", ctx)
        from .hf_loader import set_embedding

        set_embedding(model, emb)

        def fused_as_f32(layer, group):
            # gate and up share one device weight, rows interleaved, so that one GEMV applies SwiGLU on the way out.
            # A file that mixes block types inside that pair has it carried as f32 rows dequantised on the device:
            # exact, at the price of the larger read.  (q, k and v may differ: the model keeps the odd one apart;
            # llama.cpp's Q4_K_M has some attn_v in Q6_K beside Q4_K attn_q and attn_k.)
            names = [f"blk.{layer}.{_LINEAR_NAMES[w]}.weight" for w in group]
            return len({r.info(n).ggml_type for n in names}) > 1

        def linear(layer, which, name, heads=None, as_f32=False):
            if as_f32:
                from .quant import quantize_tensor

                qt = quantize_tensor(load_f32(r, name, ctx), QuantType.F32, ctx)
            else:
                qt = load_quantized_tensor(r, name, ctx)
            if heads is not None and permuted_qk:
                rows = qt.data.reshape(qt.shape[0], -1)
                qt = QuantizedTensor(qt.shape, qt.quant_type, rows[rope_rows_to_half_split(qt.shape[0], heads)])
            model.set_linear(layer, which, qt)

        for layer in range(cfg["num_hidden_layers"]):
            model.set_norm(layer, 0, load_f32(r, f"blk.{layer}.attn_norm.weight", ctx))
            model.set_norm(layer, 1, load_f32(r, f"blk.{layer}.ffn_norm.weight", ctx))
            mixed = {w: fused_as_f32(layer, g) for g in (("gate", "up"),) for w in g}
            for which, stem in _LINEAR_NAMES.items():
                heads = {"q": cfg["num_attention_heads"], "k": cfg["num_key_value_heads"]}.get(which)
                linear(layer, which, f"blk.{layer}.{stem}.weight", heads, mixed.get(which, False))
        model.set_norm(-1, 0, load_f32(r, "output_norm.weight", ctx))
        # tied embeddings: files without output.weight reuse the token embedding (llama.cpp does the same)
        linear(-1, "q", "output.weight" if "output.weight" in r.tensors else "token_embd.weight")
    return model


def tokenizer_from_metadata(md):
    """The file's vocabulary as the reference's tokenizer (`HFTokenizer`, tokenizer.rs:24-470): ids from
    `tokenizer.ggml.tokens`, merges from `tokenizer.ggml.merges` ("left right" strings, in order), special tokens from the
    `tokenizer.ggml.*_token_id` keys.  The algorithm is the reference's simple BPE, not llama.cpp's: a file whose
    `tokenizer.ggml.model` is "llama" (SentencePiece scores, no merge list) encodes to single characters or bytes."""
    from .tokenizer import HFTokenizer, SpecialTokens

    tokens = md.get("tokenizer.ggml.tokens")
    if not isinstance(tokens, (list, tuple)) or not all(isinstance(t, str) for t in tokens):
        raise GGUFError("the file has no tokenizer.ggml.tokens string array")
    vocab = {}
    for i, t in enumerate(tokens):
        vocab.setdefault(t, i)  # the first id of a repeated string, as a map built in order keeps it
    merges = []
    for m in md.get("tokenizer.ggml.merges", []) or []:
        parts = m.split(" ")
        if len(parts) == 2:
            merges.append((parts[0], parts[1]))
    special = SpecialTokens()
    for kind, key in (("bos", "bos_token_id"), ("eos", "eos_token_id"), ("unk", "unknown_token_id"), ("pad", "padding_token_id")):
        i = md.get(f"tokenizer.ggml.{key}")
        if isinstance(i, int) and 0 <= i < len(tokens):
            setattr(special, f"{kind}_token", tokens[i])
            setattr(special, f"{kind}_token_id", i)
    return HFTokenizer(vocab, {i: t for i, t in enumerate(tokens)}, merges, special, {})


def bench(ctx, log=print, n_rows=11008, k=4096, copies=8, iters=20):
    """Device-side conversion rate of a Q4_0 tensor of the 7B FFN shape (ggml order -> reference order), on
    `copies` back-to-back images so that a launch moves far more than the last-level cache holds."""
    from ._lib import MEM_DEVICE

    qt = QuantType.Q4_0
    nblocks = n_rows * k // 32 * copies
    nbytes = nblocks * qt.bytes_per_block()
    src, dst = ctx.malloc(nbytes), ctx.malloc(nbytes)
    ctx.check(ctx.lib.axq_fill_normal_f32(ctx.handle, src, nbytes // 4, 0.0, 1.0, 0.0, 0.0, 3))  # any bytes will do
    for _ in range(3):
        ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, int(qt), src, dst, nblocks, 0, MEM_DEVICE))
    ctx.synchronize()
    ctx.timer_start()
    for _ in range(iters):
        ctx.check(ctx.lib.axq_gguf_convert_blocks(ctx.handle, int(qt), src, dst, nblocks, 0, MEM_DEVICE))
    ms = ctx.timer_stop() / iters
    ctx.free(src)
    ctx.free(dst)
    res = {"type": "Q4_0", "blocks": nblocks, "bytes_read_plus_written": 2 * nbytes, "us_per_call": ms * 1e3,
           "gbps": 2 * nbytes / (ms * 1e-3) / 1e9}
    log(f"  gguf convert Q4_0, {nbytes / 1e6:.0f} MB: {ms * 1e3:.1f} us, {res['gbps']:.0f} GB/s (read + write)")
    return res
