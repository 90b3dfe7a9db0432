"""Text <-> token ids in front of and behind the decode path.

Mirrors the reference's `HFTokenizer` (crates/axonml-llm/src/tokenizer.rs:24-470), offline half:
`from_directory` (tokenizer.json, else vocab.json + merges.txt + special_tokens_map.json), `encode`,
`encode_with_options`, `decode`, `decode_with_options` and the accessors.  This is the reference's own simple
BPE, not HuggingFace's: text is cut after every whitespace or ASCII punctuation character (the cut
character stays with its piece), a piece that is a vocabulary or added token maps directly, anything
else starts as single characters and takes every merge of the list in list order, each merge applied
left to right over the whole piece; pieces without an id become the unknown token, or, when there is none,
their UTF-8 bytes as <0xNN> tokens where the vocabulary has them.  Downloads are not mirrored.
"""
import json
import os

from .hf_loader import ModelNotFound, ParseError

_ASCII_PUNCT = frozenset("!\"#$%&'()*+,-./:;<=>?@[\\]^_`{|}~")  # char::is_ascii_punctuation


class SpecialTokens:
    """SpecialTokens (tokenizer.rs:39-58): every field optional."""

    def __init__(self):
        self.bos_token = self.eos_token = self.unk_token = self.pad_token = None
        self.bos_token_id = self.eos_token_id = self.unk_token_id = self.pad_token_id = None


def _rust_whitespace(c):
    # char::is_whitespace: the Unicode White_Space property; str.isspace also accepts U+001C..U+001F
    return c.isspace() and c not in "\x1c\x1d\x1e\x1f"


def _split_inclusive(text):
    """str::split_inclusive(|c| c.is_whitespace() || c.is_ascii_punctuation()): pieces end with the
    matched character; no empty piece at the end."""
    piece = []
    for c in text:
        piece.append(c)
        if _rust_whitespace(c) or c in _ASCII_PUNCT:
            yield "".join(piece)
            piece = []
    if piece:
        yield "".join(piece)


class HFTokenizer:
    def __init__(self, vocab=None, id_to_token=None, merges=None, special_tokens=None, added_tokens=None):
        self.vocab = dict(vocab or {})
        self._id_to_token = dict(id_to_token if id_to_token is not None else {v: k for k, v in self.vocab.items()})
        self.merges = [tuple(m) for m in (merges or [])]
        self._special = special_tokens or SpecialTokens()
        self.added_tokens = dict(added_tokens or {})

    # ------------------------------------------------------------------ loading (tokenizer.rs:74-278)
    @classmethod
    def from_directory(cls, path):
        tj = os.path.join(path, "tokenizer.json")
        if os.path.exists(tj):
            return cls._load_tokenizer_json(tj)
        vj = os.path.join(path, "vocab.json")
        if os.path.exists(vj):
            return cls._load_legacy_format(vj, os.path.join(path, "merges.txt"), path)
        raise ModelNotFound("No tokenizer.json or vocab.json found")

    @staticmethod
    def _read_json(path):
        try:
            with open(path, encoding="utf-8") as f:
                return json.load(f)
        except OSError as e:
            raise ParseError(f"{path}: {e}") from None
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise ParseError(str(e)) from None

    @staticmethod
    def _as_u64(v):
        return v if isinstance(v, int) and not isinstance(v, bool) and v >= 0 else None  # serde_json's Value::as_u64

    @classmethod
    def _load_tokenizer_json(cls, path):
        doc = cls._read_json(path)
        vocab, id_to_token, merges, added = {}, {}, [], {}
        model = doc.get("model") if isinstance(doc, dict) else None
        if isinstance(model, dict):
            if isinstance(model.get("vocab"), dict):
                for token, i in model["vocab"].items():
                    if cls._as_u64(i) is not None:
                        vocab[token] = i
                        id_to_token[i] = token
            if isinstance(model.get("merges"), list):
                for m in model["merges"]:
                    if isinstance(m, str):
                        parts = m.split(" ")
                        if len(parts) == 2:
                            merges.append((parts[0], parts[1]))
        special = SpecialTokens()
        tokens = doc.get("added_tokens") if isinstance(doc, dict) else None
        if isinstance(tokens, list):
            for t in tokens:
                if not isinstance(t, dict):
                    continue
                content, i = t.get("content"), cls._as_u64(t.get("id"))
                if not isinstance(content, str) or i is None:
                    continue
                added[content] = i
                id_to_token[i] = content
                if t.get("special") is True:  # extract_special_tokens: by the look of the token's text
                    lower = content.lower()
                    if "bos" in lower or lower == "<s>":
                        special.bos_token, special.bos_token_id = content, i
                    elif "eos" in lower or lower == "</s>":
                        special.eos_token, special.eos_token_id = content, i
                    elif "unk" in lower:
                        special.unk_token, special.unk_token_id = content, i
                    elif "pad" in lower:
                        special.pad_token, special.pad_token_id = content, i
        return cls(vocab, id_to_token, merges, special, added)

    @classmethod
    def _load_legacy_format(cls, vocab_path, merges_path, directory):
        vocab = cls._read_json(vocab_path)
        if not isinstance(vocab, dict) or any(cls._as_u64(v) is None or v >= 1 << 32 for v in vocab.values()):
            raise ParseError(f"{vocab_path}: expected a map from token to u32")
        merges = []
        if os.path.exists(merges_path):
            with open(merges_path, encoding="utf-8") as f:
                for line in f.read().splitlines()[1:]:  # the first line is a header
                    parts = line.split(" ")
                    if len(parts) == 2:
                        merges.append((parts[0], parts[1]))
        special = SpecialTokens()
        sp = os.path.join(directory, "special_tokens_map.json")
        if os.path.exists(sp):
            try:
                doc = cls._read_json(sp)
            except ParseError:
                doc = None  # the reference skips a map it cannot read
            if isinstance(doc, dict):
                for kind in ("bos", "eos", "unk", "pad"):
                    t = doc.get(f"{kind}_token")
                    if isinstance(t, str):
                        setattr(special, f"{kind}_token", t)
                        setattr(special, f"{kind}_token_id", vocab.get(t))
        return cls(vocab, None, merges, special, {})

    # ------------------------------------------------------------------ encode (tokenizer.rs:280-394)
    def encode(self, text):
        return self.encode_with_options(text, True, False)

    def encode_with_options(self, text, add_bos, add_eos):
        ids = []
        if add_bos and self._special.bos_token_id is not None:
            ids.append(self._special.bos_token_id)
        ids.extend(self._bpe_encode(text))
        if add_eos and self._special.eos_token_id is not None:
            ids.append(self._special.eos_token_id)
        return ids

    def _bpe_encode(self, text):
        ids = []
        for word in _split_inclusive(text):
            if word in self.vocab:
                ids.append(self.vocab[word])
            elif word in self.added_tokens:
                ids.append(self.added_tokens[word])
            else:
                ids.extend(self._bpe_tokenize_word(word))
        return ids

    def _bpe_tokenize_word(self, word):
        parts = list(word)
        for a, b in self.merges:
            i = 0
            while i + 1 < len(parts):
                if parts[i] == a and parts[i + 1] == b:
                    parts[i:i + 2] = [a + b]  # stays at i: the merged piece may pair with the next one again
                else:
                    i += 1
        ids = []
        for part in parts:
            if part in self.vocab:
                ids.append(self.vocab[part])
            elif self._special.unk_token_id is not None:
                ids.append(self._special.unk_token_id)
            else:
                for byte in part.encode("utf-8"):
                    t = f"<0x{byte:02X}>"
                    if t in self.vocab:
                        ids.append(self.vocab[t])
        return ids

    # ------------------------------------------------------------------ decode (tokenizer.rs:396-433)
    def decode(self, ids):
        return self.decode_with_options(ids, True)

    def decode_with_options(self, ids, skip_special):
        sp = self._special
        out = []
        for i in ids:
            i = int(i)
            if skip_special and i in (sp.bos_token_id, sp.eos_token_id, sp.pad_token_id):
                continue
            token = self._id_to_token.get(i)
            if token is None:
                continue
            if token.startswith("<0x") and token.endswith(">"):
                digits = token[3:5]
                # u8::from_str_radix accepts a leading '+'; `byte as char` is the code point of that value
                if (len(digits) == 2 and all(c in "0123456789abcdefABCDEF" for c in digits)) or (
                        len(digits) == 2 and digits[0] == "+" and digits[1] in "0123456789abcdefABCDEF"):
                    out.append(chr(int(digits, 16)))
                    continue
            out.append(token)
        return "".join(out).replace("Ġ", " ").replace("▁", " ")

    # ------------------------------------------------------------------ accessors (tokenizer.rs:435-470)
    def vocab_size(self):
        return len(self.vocab) + len(self.added_tokens)

    def special_tokens(self):
        return self._special

    def bos_token_id(self):
        return self._special.bos_token_id

    def eos_token_id(self):
        return self._special.eos_token_id

    def id_to_token(self, i):
        return self._id_to_token.get(int(i))

    def token_to_id(self, token):
        return self.vocab.get(token, self.added_tokens.get(token))
