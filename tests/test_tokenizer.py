"""The reference's tokenizer (tokenizer.rs): its own unit tests, cases worked by hand from its rules,
both on-disk formats, and (GPU) text in, text out through the decode path."""
import json

import pytest

from axonml_amd import hf_loader as hf
from axonml_amd.tokenizer import HFTokenizer, SpecialTokens, _split_inclusive


def test_reference_unit_tests():
    assert SpecialTokens().bos_token is None and SpecialTokens().eos_token is None  # test_special_tokens_default
    tok = HFTokenizer({"hello": 0, " ": 1, "world": 2})
    assert tok.decode([0, 1, 2]) == "hello world"                                     # test_bpe_simple
    tok = HFTokenizer({"a": 0, "b": 1}, id_to_token={}, added_tokens={"<special>": 2})
    assert tok.vocab_size() == 3                                                      # test_vocab_size


def test_split_keeps_the_cut_character_with_its_piece():
    assert list(_split_inclusive("hello world")) == ["hello ", "world"]
    assert list(_split_inclusive("a,b  c!")) == ["a,", "b ", " ", "c!"]
    assert list(_split_inclusive("")) == []
    assert list(_split_inclusive("x\n")) == ["x\n"]
    assert list(_split_inclusive("don't")) == ["don'", "t"]
    assert list(_split_inclusive("a b　c")) == ["a ", "b　", "c"]  # Unicode white space cuts
    assert list(_split_inclusive("a\x1cb—c")) == ["a\x1cb—c"]                # U+001C and a dash outside ASCII do not


def test_merges_apply_in_list_order_each_over_the_whole_piece():
    vocab = {"l": 0, "o": 1, "w": 2, "lo": 3, "low": 4, "e": 5, "r": 6, "er": 7, "ow": 8, " ": 9, "lower": 10}
    # "lower" is a vocabulary entry: direct hit, no BPE
    assert HFTokenizer(vocab, merges=[("l", "o")]).encode("lower") == [10]
    del vocab["lower"]
    # l o w e r --(l,o)--> lo w e r --(lo,w)--> low e r --(e,r)--> low er
    assert HFTokenizer(vocab, merges=[("l", "o"), ("lo", "w"), ("e", "r")]).encode("lower") == [4, 7]
    # list order decides, not adjacency: (o,w) first takes the w, so (lo,w) never fires
    assert HFTokenizer(vocab, merges=[("o", "w"), ("l", "o"), ("lo", "w"), ("e", "r")]).encode("lower") == [0, 8, 7]
    # the piece keeps its trailing space ("low " is no vocabulary entry), which stays a character of its own
    assert HFTokenizer(vocab, merges=[("l", "o"), ("lo", "w")]).encode("low lo") == [4, 9, 3]
    # a merged piece is looked at again at the same place: aaaa -> aa a a -> aa aa
    t = HFTokenizer({"a": 0, "aa": 1}, merges=[("a", "a")])
    assert t.encode("aaaa") == [1, 1] and t.encode("aaa") == [1, 0]
    t = HFTokenizer({"a": 0, "aa": 1, "aaa": 2}, merges=[("a", "a"), ("aa", "a")])
    assert t.encode("aaaa") == [1, 1] and t.encode("aaaaa") == [1, 2]  # aa aa stays; aa aa a -> aa aaa


def test_unknown_pieces():
    vocab = {"a": 0, "<unk>": 1}
    sp = SpecialTokens()
    sp.unk_token, sp.unk_token_id = "<unk>", 1
    assert HFTokenizer(vocab, special_tokens=sp).encode("abz") == [0, 1, 1]
    # no unknown token: UTF-8 bytes as <0xNN> where the vocabulary has them, nothing otherwise
    vocab = {"a": 0, "<0xC3>": 5, "<0xA9>": 6, "<0x62>": 7}
    assert HFTokenizer(vocab).encode("aébz") == [0, 5, 6, 7]


def test_bos_eos_options():
    sp = SpecialTokens()
    sp.bos_token_id, sp.eos_token_id = 1, 2
    t = HFTokenizer({"hi": 5}, special_tokens=sp)
    assert t.encode("hi") == [1, 5]  # encode adds the beginning, never the end
    assert t.encode_with_options("hi", False, False) == [5]
    assert t.encode_with_options("hi", True, True) == [1, 5, 2]
    assert HFTokenizer({"hi": 5}).encode_with_options("hi", True, True) == [5]  # none configured, none added
    assert t.bos_token_id() == 1 and t.eos_token_id() == 2


def test_decode_rules():
    sp = SpecialTokens()
    sp.bos_token_id, sp.eos_token_id, sp.pad_token_id, sp.unk_token_id = 0, 1, 2, 3
    vocab = {"<s>": 0, "</s>": 1, "<pad>": 2, "<unk>": 3, "▁Hello": 4, "Ġworld": 5, "<0x41>": 6, "<0xE9>": 7, "<0xZZ>": 8}
    t = HFTokenizer(vocab, special_tokens=sp)
    assert t.decode([0, 4, 5, 1, 2]) == " Hello world"
    assert t.decode_with_options([0, 4, 1], False) == "<s> Hello</s>"
    assert t.decode([3]) == "<unk>"                     # the unknown token is not skipped
    assert t.decode([6, 7]) == "Aé"                # `byte as char`: the code point, not a UTF-8 byte
    assert t.decode([8, 99]) == "<0xZZ>"                # not hexadecimal: kept as text; unknown ids are dropped
    assert t.id_to_token(4) == "▁Hello" and t.id_to_token(99) is None
    assert t.token_to_id("<pad>") == 2 and t.token_to_id("nope") is None


def _tokenizer_json():
    return {"model": {"type": "BPE", "vocab": {"h": 0, "i": 1, "hi": 2, " ": 3, "!": 4, "bad": "x"},
                      "merges": ["h i", "too many parts", 7]},
            "added_tokens": [{"id": 10, "content": "<s>", "special": True}, {"id": 11, "content": "</s>", "special": True},
                             {"id": 12, "content": "<|unk|>", "special": True}, {"id": 13, "content": "[PAD]", "special": True},
                             {"id": 14, "content": "<extra>", "special": False}, {"id": 15, "content": "<custom>", "special": True},
                             {"content": "no id"}]}


def test_tokenizer_json(tmp_path):
    (tmp_path / "tokenizer.json").write_text(json.dumps(_tokenizer_json()))
    (tmp_path / "vocab.json").write_text("{}")  # ignored when tokenizer.json is there
    t = HFTokenizer.from_directory(str(tmp_path))
    assert t.vocab == {"h": 0, "i": 1, "hi": 2, " ": 3, "!": 4} and t.merges == [("h", "i")]
    assert t.added_tokens == {"<s>": 10, "</s>": 11, "<|unk|>": 12, "[PAD]": 13, "<extra>": 14, "<custom>": 15}
    sp = t.special_tokens()
    assert (sp.bos_token, sp.bos_token_id, sp.eos_token, sp.eos_token_id) == ("<s>", 10, "</s>", 11)
    assert (sp.unk_token_id, sp.pad_token_id) == (12, 13)
    assert t.vocab_size() == 11
    assert t.encode("hi hi!") == [10, 2, 3, 2, 4]  # "hi " -> h i ' ' -> hi ' '; "hi!" -> hi !
    assert t.encode("<extra>") == [10, 12, 12, 12, 12, 12, 12, 12]  # cut after '<' ... '>' never matches the added token: all unknown
    assert t.encode_with_options("hi</s>", False, False) == [2, 12, 12, 12, 12]  # "hi<", "/", "s>"
    assert t.decode([10, 2, 3, 14, 11]) == "hi <extra>"
    assert t.token_to_id("<custom>") == 15


def test_legacy_format(tmp_path):
    (tmp_path / "vocab.json").write_text(json.dumps({"a": 0, "b": 1, "ab": 2, "<|endoftext|>": 3, "Ġ": 4}))
    (tmp_path / "merges.txt").write_text("#version: 0.2\na b\nbroken line here\n\n")
    (tmp_path / "special_tokens_map.json").write_text(json.dumps(
        {"bos_token": "<|endoftext|>", "eos_token": "<|endoftext|>", "unk_token": "<|endoftext|>", "pad_token": {"content": "x"}}))
    t = HFTokenizer.from_directory(str(tmp_path))
    assert t.merges == [("a", "b")] and t.added_tokens == {}
    sp = t.special_tokens()
    assert sp.bos_token_id == 3 and sp.eos_token_id == 3 and sp.unk_token_id == 3 and sp.pad_token_id is None
    assert t.encode("abab") == [3, 2, 2]
    assert t.decode([3, 2, 4, 0]) == "ab a"
    # without the optional files
    (tmp_path / "merges.txt").unlink()
    (tmp_path / "special_tokens_map.json").write_text("{ not json")
    t = HFTokenizer.from_directory(str(tmp_path))
    assert t.merges == [] and t.bos_token_id() is None and t.encode("ab") == [2] and t.encode("ba") == [1, 0]


def test_loading_errors(tmp_path):
    with pytest.raises(hf.ModelNotFound, match="No tokenizer.json or vocab.json"):
        HFTokenizer.from_directory(str(tmp_path))
    (tmp_path / "tokenizer.json").write_text("{ nope")
    with pytest.raises(hf.ParseError):
        HFTokenizer.from_directory(str(tmp_path))
    (tmp_path / "tokenizer.json").unlink()
    (tmp_path / "vocab.json").write_text(json.dumps({"a": -1}))
    with pytest.raises(hf.ParseError):
        HFTokenizer.from_directory(str(tmp_path))
    (tmp_path / "vocab.json").write_text(json.dumps({"a": 1}))
    (tmp_path / "tokenizer.json").write_text(json.dumps({"model": 3, "added_tokens": "x"}))  # odd shapes are skipped, not errors
    t = HFTokenizer.from_directory(str(tmp_path))
    assert t.vocab == {} and t.vocab_size() == 0 and t.encode("a") == []


@pytest.mark.gpu
def test_text_through_the_decode_path(ctx, tmp_path):
    """Text -> ids -> prompt fed at once and greedy generation on the device -> text, against the oracle's walk."""
    import oracle as o
    from tests.decode_common import load_gpu, load_oracle, random_weights, tiny_config

    c = tiny_config()
    words = ["the ", "quick ", "brown ", "fox ", "jumps ", "over ", "lazy ", "dog.", " ", "a", "b", "c"]
    vocab = {w: i + 2 for i, w in enumerate(words)}
    vocab.update({f"t{i}": i for i in range(len(words) + 2, c["vocab_size"])})
    doc = {"model": {"vocab": vocab, "merges": []},
           "added_tokens": [{"id": 0, "content": "<s>", "special": True}, {"id": 1, "content": "</s>", "special": True}]}
    (tmp_path / "tokenizer.json").write_text(json.dumps(doc))
    tok = HFTokenizer.from_directory(str(tmp_path))
    ids = tok.encode("the quick brown fox jumps over the lazy dog. abc")
    assert ids == [0, 2, 3, 4, 5, 6, 7, 2, 8, 9, 10, 11, 12, 13]
    w = random_weights(c, 77)
    cpu, gpu = load_oracle(c, w), load_gpu(ctx, c, w)
    for pos, t in enumerate(ids):
        nxt, _ = cpu.forward(t, pos)
    want = []
    for i in range(12):
        want.append(nxt)
        if i + 1 < 12:
            nxt, _ = cpu.forward(nxt, len(ids) + i)
    got, _, _ = gpu.generate(ids, 12)
    assert got.tolist() == want
    assert tok.decode(got) == "".join(tok.id_to_token(i) for i in want if i not in (0, 1))
    gpu.close()
