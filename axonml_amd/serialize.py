"""State dictionaries on disk, with an entry for quantized tensors.

Mirrors the reference's `StateDict` / `StateDictEntry` / `TensorData` (crates/axonml-serialize/src/state_dict.rs:15-260)
and `save_state_dict` / `load_state_dict` / `detect_format` (src/lib.rs:120-210, src/format.rs:79-92) for its two
default-feature formats:

* Axonml native (.axonml, .bin, anything else): `bincode::serialize(&StateDict)`, bincode 1.3 with its legacy
  options: little-endian, fixed-width integers, usize and every length as u64, f32 as 4 bytes, bool as one
  byte, String = length + UTF-8, Vec = length + items, HashMap = length + (key, value) pairs, struct fields
  in declaration order.
* JSON (.json): `serde_json::to_writer_pretty` of the same struct.

The reference's `TensorData` is f32 only (state_dict.rs:17-22), so its `axonml quant convert` writes
f32 copies (cli/src/commands/quant.rs:171-180, 236-260).  The entry added here keeps a quantized tensor as
what `QuantizedTensor` is: type tag, shape, and the block images in `to_bytes` order (types.rs:320-335):

* native: after the StateDict's bytes comes `bincode(Vec<(String, QuantizedTensorData)>)` with
  `QuantizedTensorData { quant_type: u32, shape: Vec<usize>, data: Vec<u8> }`, then 16 bytes of footer:
  b"AXQTENS1" and the u64 offset of that section.  `bincode::deserialize` of the legacy API ignores bytes
  after the value it reads, so the reference's own `load_state_dict` still loads the f32 entries of such a
  file and never sees the rest.
* JSON: a third top-level key "quantized": {name: {"quant_type": "Q4_K", "shape": [..], "data": [bytes]}};
  serde ignores unknown keys unless told otherwise.
"""
import json
import os
import struct

import numpy as np

from .quant import QuantError, QuantizedTensor, QuantType

FOOTER_MAGIC = b"AXQTENS1"


class SerializeError(QuantError):
    """Error::InvalidOperation of the serializer (lib.rs:120-210 maps every failure to it)."""


# --------------------------------------------------------------------------- format detection (format.rs)
class Format:
    Axonml, Json, SafeTensors = "Axonml Native", "JSON", "SafeTensors"
    _EXT = {Axonml: "axonml", Json: "json", SafeTensors: "safetensors"}

    @staticmethod
    def extension(fmt):
        return Format._EXT[fmt]

    @staticmethod
    def is_binary(fmt):
        return fmt != Format.Json

    @staticmethod
    def all():
        return [Format.Axonml, Format.Json, Format.SafeTensors]


def detect_format(path):
    """detect_format (format.rs:79-92): by extension, case-sensitive, native by default."""
    ext = os.path.basename(str(path)).rpartition(".")
    ext = ext[2] if ext[1] and ext[0] else None  # Path::extension: none for "name" and for ".hidden"
    return {"axonml": Format.Axonml, "bin": Format.Axonml, "json": Format.Json, "safetensors": Format.SafeTensors,
            "st": Format.SafeTensors}.get(ext, Format.Axonml)


def detect_format_from_bytes(data):
    """detect_format_from_bytes (format.rs:95-119)."""
    if len(data) < 8:
        return None
    if data[0] in b"{[":
        return Format.Json
    if len(data) >= 16:
        (n,) = struct.unpack("<Q", data[:8])
        if n < 10_000_000 and data[8:9] == b"{":
            return Format.SafeTensors
    return Format.Axonml


# --------------------------------------------------------------------------- the structs
class TensorData:
    """TensorData (state_dict.rs:15-50): shape and flattened f32 values."""

    def __init__(self, shape, values):
        self.shape = [int(s) for s in shape]
        self.values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)

    @classmethod
    def from_tensor(cls, tensor):
        t = np.asarray(tensor, dtype=np.float32)
        return cls(t.shape, t)

    def to_tensor(self):
        n = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        if n != self.values.size:  # Tensor::from_vec refuses a length that does not match the shape
            raise SerializeError(f"shape {self.shape} does not hold {self.values.size} values")
        return self.values.reshape(self.shape)

    def numel(self):
        return int(self.values.size)


class StateDictEntry:
    """StateDictEntry (state_dict.rs:56-85)."""

    def __init__(self, data, requires_grad=True, metadata=None):
        self.data, self.requires_grad, self.metadata = data, bool(requires_grad), dict(metadata or {})

    def with_metadata(self, key, value):
        self.metadata[str(key)] = str(value)
        return self


class StateDict:
    """StateDict (state_dict.rs:94-260) plus `quantized`: name -> QuantizedTensor."""

    def __init__(self):
        self.entries, self.metadata, self.quantized = {}, {}, {}

    # the reference's methods
    def insert(self, name, data):
        self.entries[name] = StateDictEntry(data, True)

    def insert_entry(self, name, entry):
        self.entries[name] = entry

    def get(self, name):
        return self.entries.get(name)

    def contains(self, name):
        return name in self.entries

    def __len__(self):
        return len(self.entries)

    def is_empty(self):
        return not self.entries

    def keys(self):
        return self.entries.keys()

    def remove(self, name):
        return self.entries.pop(name, None)

    def merge(self, other):
        self.entries.update(other.entries)
        self.quantized.update(other.quantized)

    def _renamed(self, keep, rename):
        out = StateDict()
        for src, dst in ((self.entries, out.entries), (self.quantized, out.quantized)):
            for name, e in src.items():
                if keep(name):
                    dst[rename(name)] = e
        return out

    def filter_prefix(self, prefix):
        return self._renamed(lambda n: n.startswith(prefix), lambda n: n)

    def strip_prefix(self, prefix):
        return self._renamed(lambda n: True, lambda n: n[len(prefix):] if n.startswith(prefix) else n)

    def add_prefix(self, prefix):
        return self._renamed(lambda n: True, lambda n: prefix + n)

    def set_metadata(self, key, value):
        self.metadata[str(key)] = str(value)

    def get_metadata(self, key):
        return self.metadata.get(key)

    def total_params(self):
        return sum(e.data.numel() for e in self.entries.values())

    def size_bytes(self):
        return self.total_params() * 4

    def summary(self):
        lines = [f"StateDict with {len(self)} entries:", f"  Total parameters: {self.total_params()}",
                 f"  Size: {self.size_bytes()} bytes", "  Entries:"]
        for name, e in self.entries.items():
            lines.append(f"    {name} - shape: {e.data.shape}, numel: {e.data.numel()}")
        return "\n".join(lines)

    # the quantized entries
    def insert_quantized(self, name, tensor):
        if not isinstance(tensor, QuantizedTensor):
            raise TypeError("insert_quantized takes a QuantizedTensor")
        self.quantized[name] = tensor

    def get_quantized(self, name):
        return self.quantized.get(name)

    def quantized_bytes(self):
        return sum(int(t.data.size) for t in self.quantized.values())


# --------------------------------------------------------------------------- bincode 1.3, legacy options
class _Writer:
    def __init__(self):
        self.parts = []

    def u64(self, v):
        self.parts.append(struct.pack("<Q", v))

    def string(self, s):
        b = s.encode("utf-8")
        self.u64(len(b))
        self.parts.append(b)

    def string_map(self, m):
        self.u64(len(m))
        for k, v in m.items():
            self.string(k)
            self.string(v)

    def usize_vec(self, v):
        self.u64(len(v))
        self.parts.append(np.asarray(v, dtype="<u8").tobytes())


class _Reader:
    def __init__(self, buf, pos=0, end=None):
        self.buf, self.pos, self.end = buf, pos, len(buf) if end is None else end

    def take(self, n):
        if n < 0 or self.pos + n > self.end:
            raise SerializeError("io error: unexpected end of file")  # bincode's ErrorKind::Io(UnexpectedEof)
        p = self.pos
        self.pos += n
        return p

    def u64(self):
        return struct.unpack_from("<Q", self.buf, self.take(8))[0]

    def u32(self):
        return struct.unpack_from("<I", self.buf, self.take(4))[0]

    def boolean(self):
        b = self.buf[self.take(1)]
        if b > 1:
            raise SerializeError(f"invalid u8 while decoding bool, expected 0 or 1, found {b}")
        return bool(b)

    def string(self):
        n = self.u64()
        p = self.take(n)
        try:
            return bytes(self.buf[p:p + n]).decode("utf-8")
        except UnicodeDecodeError as e:
            raise SerializeError(f"string is not valid utf8: {e}") from None

    def string_map(self):
        return {self.string(): self.string() for _ in range(self._count(16))}

    def _count(self, min_item_bytes):
        n = self.u64()
        if n * min_item_bytes > self.end - self.pos:  # a length that the rest of the file cannot hold
            raise SerializeError("io error: unexpected end of file")
        return n

    def array(self, dtype, width):
        n = self._count(width)
        p = self.take(n * width)
        return np.frombuffer(self.buf, dtype=dtype, count=n, offset=p)


def _encode_state_dict(sd):
    w = _Writer()
    w.u64(len(sd.entries))
    for name, e in sd.entries.items():
        w.string(name)
        w.usize_vec(e.data.shape)
        w.u64(e.data.values.size)
        w.parts.append(e.data.values.astype("<f4", copy=False).tobytes())
        w.parts.append(b"\x01" if e.requires_grad else b"\x00")
        w.string_map(e.metadata)
    w.string_map(sd.metadata)
    return w.parts


def _encode_quantized(sd):
    w = _Writer()
    w.u64(len(sd.quantized))
    for name, t in sd.quantized.items():
        w.string(name)
        w.parts.append(struct.pack("<I", int(t.quant_type)))
        w.usize_vec(t.shape)
        w.u64(t.data.size)
        w.parts.append(t.data.tobytes())
    return w.parts


def _decode_state_dict(r, sd):
    for _ in range(r._count(8 + 8 + 8 + 1 + 8)):
        name = r.string()
        shape = [int(v) for v in r.array("<u8", 8)]
        values = r.array("<f4", 4).astype(np.float32)
        requires_grad = r.boolean()
        sd.entries[name] = StateDictEntry(TensorData(shape, values), requires_grad, r.string_map())
    sd.metadata = r.string_map()


def _decode_quantized(r, sd):
    for _ in range(r._count(8 + 4 + 8 + 8)):
        name = r.string()
        tag = r.u32()
        shape = [int(v) for v in r.array("<u8", 8)]
        data = r.array(np.uint8, 1)
        try:
            qt = QuantType(tag)
        except ValueError:
            raise SerializeError(f"entry {name}: unknown quantization type tag {tag}") from None
        sd.quantized[name] = QuantizedTensor(shape, qt, data.copy())  # checks the byte count against the shape


# --------------------------------------------------------------------------- JSON
def _json_f32(values):
    out = []
    for v in values:
        out.append(str(v) if np.isfinite(v) else "null")  # numpy prints the shortest digits that give the f32 back, as ryu does
    return "[" + ", ".join(out) + "]"


def _encode_json(sd):
    entries = []
    for name, e in sd.entries.items():
        entries.append(f'    {json.dumps(name)}: {{\n      "data": {{"shape": {json.dumps(e.data.shape)}, "values": {_json_f32(e.data.values)}}},\n'
                       f'      "requires_grad": {"true" if e.requires_grad else "false"},\n      "metadata": {json.dumps(e.metadata)}\n    }}')
    text = '{\n  "entries": {\n' + ",\n".join(entries) + '\n  },\n  "metadata": ' + json.dumps(sd.metadata)
    if sd.quantized:
        q = {name: {"quant_type": str(t.quant_type), "shape": t.shape, "data": t.data.tolist()} for name, t in sd.quantized.items()}
        text += ',\n  "quantized": ' + json.dumps(q)
    return text + "\n}\n"


def _decode_json(text, sd):
    try:
        doc = json.loads(text)
        for name, e in doc["entries"].items():
            values = e["data"]["values"]
            if any(v is None for v in values):
                raise SerializeError(f"entry {name}: invalid type: null, expected f32")
            sd.entries[name] = StateDictEntry(TensorData(e["data"]["shape"], values), e["requires_grad"], e.get("metadata", {}))
        sd.metadata = dict(doc.get("metadata", {}))
        for name, e in doc.get("quantized", {}).items():
            qt = QuantType.from_str(e["quant_type"])
            if qt is None:
                raise SerializeError(f"entry {name}: unknown quantization type {e['quant_type']}")
            sd.quantized[name] = QuantizedTensor(e["shape"], qt, np.asarray(e["data"], dtype=np.uint8))
    except (json.JSONDecodeError, KeyError, TypeError, ValueError) as err:
        raise SerializeError(str(err)) from None


# --------------------------------------------------------------------------- save / load (lib.rs:120-210)
def save_state_dict(state_dict, path, fmt=None):
    fmt = fmt or detect_format(path)
    if fmt == Format.SafeTensors:  # the reference's default build (lib.rs:152-157)
        raise SerializeError("SafeTensors format requires 'safetensors' feature")
    try:
        if fmt == Format.Json:
            with open(path, "w", encoding="utf-8") as f:
                f.write(_encode_json(state_dict))
            return
        with open(path, "wb") as f:
            offset = 0
            for part in _encode_state_dict(state_dict):
                f.write(part)
                offset += len(part)
            if state_dict.quantized:
                for part in _encode_quantized(state_dict):
                    f.write(part)
                f.write(FOOTER_MAGIC + struct.pack("<Q", offset))
    except OSError as e:
        raise SerializeError(str(e)) from None


def load_state_dict(path):
    fmt = detect_format(path)
    if fmt == Format.SafeTensors:
        raise SerializeError("SafeTensors format requires 'safetensors' feature")
    sd = StateDict()
    try:
        if fmt == Format.Json:
            with open(path, encoding="utf-8") as f:
                _decode_json(f.read(), sd)
            return sd
        buf = np.fromfile(path, dtype=np.uint8)
    except OSError as e:
        raise SerializeError(str(e)) from None
    mem = memoryview(buf)
    r = _Reader(mem)
    _decode_state_dict(r, sd)
    if len(buf) >= r.pos + 16 and bytes(mem[-16:-8]) == FOOTER_MAGIC:
        (offset,) = struct.unpack("<Q", mem[-8:])
        if offset != r.pos:
            raise SerializeError(f"quantized section at {offset}, but the state dictionary ends at {r.pos}")
        q = _Reader(mem, offset, len(buf) - 16)
        _decode_quantized(q, sd)
        if q.pos != q.end:
            raise SerializeError("trailing bytes in the quantized section")
    return sd


# --------------------------------------------------------------------------- quantize a state dictionary
def quantize_state_dict(state_dict, quant_type, ctx=None, min_dims=2):
    """What `axonml quant convert` sets out to do (cli/src/commands/quant.rs:236-260): every entry of at
    least `min_dims` dimensions becomes a quantized entry (on the device, `quantize_tensor`,
    quantize.rs:36-54); vectors (norm weights, biases) stay f32."""
    from .quant import quantize_tensor

    out = StateDict()
    out.metadata = dict(state_dict.metadata)
    out.quantized = dict(state_dict.quantized)
    for name, e in state_dict.entries.items():
        if len(e.data.shape) >= min_dims:
            out.quantized[name] = quantize_tensor(e.data.to_tensor(), quant_type, ctx)
        else:
            out.entries[name] = e
    return out
