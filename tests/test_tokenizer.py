"""The text front end (CPU only): reference vectors -> oracle and library; library vs oracle on generated text;
the library's Unicode tables vs Python's unicodedata."""
import json
import os
import random
import unicodedata

import numpy as np
import pytest

import cubert_amd
from cubert_amd._lib import lib
from oracle import tokenizer as otok

HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = json.load(open(os.path.join(HERE, "golden", "tokenization_vectors.json"), encoding="utf8"))


@pytest.fixture(scope="module")
def vocab_file(tmp_path_factory):
    """The reference's 11-line test vocabulary (test_vocab.txt), rewritten from the fixture."""
    path = tmp_path_factory.mktemp("vocab") / "test_vocab.txt"
    path.write_text("\n".join(VECTORS["test_vocab"]) + "\n", encoding="utf8")
    return str(path)


class _Runner(object):
    """Replays the steps of one reference TEST_F against an implementation."""

    def __init__(self, tokenize, token_id):
        self.tokenize, self.token_id, self.tokens = tokenize, token_id, []

    def run(self, steps):
        checked = 0
        for s in steps:
            if s["op"] == "tokenize":
                self.tokens += self.tokenize(s["text"], s["max_length"])
            elif s["op"] == "clear":
                self.tokens = []
            elif s["op"] == "set":
                self.tokens = list(s["tokens"])
            elif s["op"] == "expect_token":
                assert self.tokens[s["index"]] == s["token"], (s, self.tokens)
                checked += 1
            elif s["op"] == "expect_size":
                assert len(self.tokens) == s["size"]
                checked += 1
            elif s["op"] == "expect_id":
                assert self.token_id(self.tokens[s["index"]]) == s["id"], (s, self.tokens)
                checked += 1
        return checked


def _implementations(test, vocab_file):
    """(name, tokenize(text, max_length) -> tokens, token_id) for the oracle and for the library."""
    vocab = otok.load_vocab(VECTORS["test_vocab"])
    receiver, args = test["receiver"], test["constructor_args"]
    lower = args != "false"
    if receiver == "BasicTokenizer":
        lib_tok = cubert_amd.Tokenizer(None, do_lower_case=lower)
        return [("oracle", lambda t, n: otok.basic_tokenize(t, lower, n), None),
                ("library", lambda t, n: lib_tok.tokenize(t, n), None)]
    lib_tok = cubert_amd.Tokenizer(vocab_file, do_lower_case=True)
    if receiver == "WordpieceTokenizer":
        return [("oracle", lambda t, n: otok.wordpiece(t, vocab), vocab.get),
                ("library", lambda t, n: lib_tok.wordpiece(t), None)]
    return [("oracle", lambda t, n: otok.full_tokenize(t, vocab, True, n), lambda t: vocab.get(t, 0)),
            ("library", lambda t, n: lib_tok.tokenize(t, n), lambda t: lib_tok.convert_tokens_to_ids([t])[0])]


@pytest.mark.parametrize("name", sorted(k for k, v in VECTORS["tests"].items() if v["steps"]))
def test_reference_tokenizer_vectors(name, vocab_file):
    """test/cuBERT/tokenization_test.cpp:12-124 of the reference, every EXPECT, on both implementations."""
    test = VECTORS["tests"][name]
    for impl, tokenize, token_id in _implementations(test, vocab_file):
        assert _Runner(tokenize, token_id).run(test["steps"]) > 0, impl


def test_reference_character_class_vectors():
    """test/cuBERT/tokenization_test.cpp:126-152."""
    which = {"_is_whitespace": 0, "_is_control": 1, "_is_punctuation": 2}
    oracle_fn = {"_is_whitespace": otok.is_whitespace, "_is_control": otok.is_control,
                 "_is_punctuation": otok.is_punctuation}
    n = 0
    for test in VECTORS["tests"].values():
        for c in test["char_classes"]:
            assert oracle_fn[c["function"]](c["code_point"]) == c["expect"], c
            assert bool(lib().cubert_tokenizer_char_class(which[c["function"]], c["code_point"])) == c["expect"], c
            n += 1
    assert n == 18


def test_unicode_tables_match_unicodedata():
    """Character classes and simple lower-casing (through the basic tokenizer) of every code point, and the
    decomposition of every code point that has one, against Python's unicodedata of the same Unicode version."""
    L = lib()
    assert L.cubert_tokenizer_unicode_version().decode() == unicodedata.unidata_version
    for cp in list(range(0, 0x3400)) + list(range(0x4DB0, 0x4E10)) + list(range(0x9FF0, 0x31400, 1)) + \
            list(range(0xE0000, 0xE0200)) + [0xEFFFF, 0xF0000, 0x10FFFD, 0x10FFFF]:
        assert bool(L.cubert_tokenizer_char_class(0, cp)) == otok.is_whitespace(cp), hex(cp)
        assert bool(L.cubert_tokenizer_char_class(1, cp)) == otok.is_control(cp), hex(cp)
        assert bool(L.cubert_tokenizer_char_class(2, cp)) == otok.is_punctuation(cp), hex(cp)
    # NFD: batches of code points separated by 'a' (a starter, so marks do not reorder across it)
    cps = [cp for cp in range(0x80, 0x110000) if not 0xD800 <= cp <= 0xDFFF]
    for i in range(0, len(cps), 4096):
        s = "a".join(chr(cp) for cp in cps[i:i + 4096])
        assert cubert_amd.nfd(s) == unicodedata.normalize("NFD", s), hex(cps[i])
    # lower-casing: every cased letter as a one-character text
    basic = cubert_amd.Tokenizer(None, do_lower_case=True)
    letters = [cp for cp in range(0x41, 0x1F000) if unicodedata.category(chr(cp)) in ("Lu", "Lt")]
    text = " ".join(chr(cp) for cp in letters)
    assert basic.tokenize(text) == otok.basic_tokenize(text, True)


def test_nfd_reorders_marks():
    """Canonical ordering: marks of different combining classes are sorted, equal classes keep their order."""
    for s in ["à֮̀̕b", "ḍ̇", "Ḕ́", "한글", "q̣̇",
              "ཱཱིི", "ǖͅ"]:
        assert cubert_amd.nfd(s) == unicodedata.normalize("NFD", s), ascii(s)


ALPHABET = (
    [chr(c) for c in range(0x20, 0x7F)] * 3 + list("\t\n\r") +
    [chr(c) for c in range(0xA0, 0x180)] +                        # Latin-1 / Latin Extended-A (accents, nbsp, soft hyphen)
    [chr(c) for c in range(0x300, 0x330)] +                       # combining marks
    list("ΑΒΣσςΩάΐ" "ЖжЁё" "İıǅǆ" "ẞß") +
    list("博推知乎发现更大的世界") + ["㐀", "\U00020000", "豈", "\U0002F800"] +
    list("한글가힣") + list("あア々〆") + ["　", " ", "​", "‍", "﻿", "\u0085", " "] +
    list("—…“”«»、。！？¿¡") + ["�", "\u0001", "\u007F", "\U0001F600", "", "͸", "\U000E0001"]
)


def _random_text(rng, n):
    return "".join(rng.choice(ALPHABET) for _ in range(n))


@pytest.mark.parametrize("lower", [True, False])
def test_basic_tokenizer_matches_oracle_on_generated_text(lower):
    rng = random.Random(1234 + lower)
    basic = cubert_amd.Tokenizer(None, do_lower_case=lower)
    for i in range(400):
        text = _random_text(rng, rng.randint(0, 120))
        limit = rng.choice([1, 2, 5, 32, 1000])
        assert basic.tokenize(text, limit) == otok.basic_tokenize(text, lower, limit), ascii(text)


def test_full_tokenizer_and_examples_match_oracle(tmp_path):
    """A vocabulary cut out of generated text (so word pieces, '##' continuations and [UNK] all occur), then texts
    and text pairs through tokenize and convert_single_example with several sequence lengths."""
    rng = random.Random(7)
    corpus = [_random_text(rng, rng.randint(1, 80)) for _ in range(300)]
    pieces = {"[UNK]", "[CLS]", "[SEP]", "[PAD]"}
    for text in corpus[:200]:
        for tok in otok.basic_tokenize(text, True):
            raw = tok.encode("utf8")
            cut = rng.randint(1, len(raw))
            for a, b in ((0, cut), (cut, len(raw))):
                try:
                    piece = raw[a:b].decode("utf8")
                except UnicodeDecodeError:
                    continue
                if piece and rng.random() < 0.7:
                    pieces.add(("##" if a else "") + piece)
    lines = ["[PAD]"] + sorted(pieces - {"[PAD]"})
    path = tmp_path / "vocab.txt"
    path.write_text("\n".join(lines) + "\n", encoding="utf8")
    vocab = otok.load_vocab(lines)
    tok = cubert_amd.Tokenizer(str(path))
    unk = 0
    for text in corpus:
        want = otok.full_tokenize(text, vocab, True, 64)
        assert tok.tokenize(text, 64) == want, ascii(text)
        assert tok.convert_tokens_to_ids(want) == [vocab.get(t, 0) for t in want]
        unk += want.count("[UNK]")
    assert unk > 0
    for i in range(0, len(corpus) - 1, 2):
        for seq in (8, 16, 32, 128):
            for b in (None, corpus[i + 1]):
                ids, mask, seg = tok.convert_example(seq, corpus[i], b)
                w_ids, w_mask, w_seg = otok.convert_single_example(vocab, seq, corpus[i], b)
                assert ids.tolist() == w_ids and mask.tolist() == w_mask and seg.tolist() == w_seg, (seq, ascii(corpus[i]))


def test_edge_cases(vocab_file):
    tok = cubert_amd.Tokenizer(vocab_file)
    basic = cubert_amd.Tokenizer(None)
    assert tok.tokenize("") == [] and basic.tokenize("  \t\n ") == []
    # a token of more than 200 bytes is unknown as a whole (tokenization.cpp:187-190); 200 bytes are still split
    assert tok.tokenize("un" * 101) == ["[UNK]"]
    assert tok.wordpiece("un" + "wa" * 0) == ["un"]
    # text after malformed UTF-8 is dropped (tokenization.cpp:133-137)
    assert basic.tokenize(b"ab cd\xff ef") == ["ab", "cd"] == otok.basic_tokenize(b"ab cd\xff ef")
    assert basic.tokenize(b"ab \xe4\xb8") == ["ab"]
    assert basic.tokenize(b"\xc0\xaf overlong") == [] and basic.tokenize(b"\xed\xa0\x80 surrogate") == []
    # the token that reaches max_length keeps only its first character (tokenization.cpp:175-178)
    assert basic.tokenize("one two three", 2) == ["one", "t"] == otok.basic_tokenize("one two three", True, 2)
    # an unknown token has id 0 (tokenization.h:131-139)
    assert tok.convert_tokens_to_ids(["nope", "un"]) == [0, 7]
    # pair truncation drops from the longer sequence, from b on a tie (cuBERT.cpp:118-135)
    ids, mask, seg = tok.convert_example(8, "unwanted running ,", "running , wa un")
    # a: 6 pieces, b: 5 pieces, 5 fit -> a keeps 3, b keeps 2: [CLS] a a a [SEP] b b [SEP]
    assert mask.tolist() == [1] * 8 and seg.tolist() == [0, 0, 0, 0, 0, 1, 1, 1]
    assert ids.tolist() == [1, 7, 4, 5, 2, 8, 9, 2]
    vocab = otok.load_vocab(VECTORS["test_vocab"])
    assert otok.convert_single_example(vocab, 8, "unwanted running ,", "running , wa un")[0] == ids.tolist()
    with pytest.raises(ValueError):
        tok.convert_example(1, "un")
    with pytest.raises(ValueError):
        cubert_amd.Tokenizer("/nonexistent/vocab.txt")
