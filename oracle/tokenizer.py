"""CPU restatement of the reference's text front end, for tests only.

Follows src/cuBERT/tokenization.cpp of the reference function by function, with Python's `unicodedata` in the
place of utf8proc (NFD: tokenization.cpp:123-125; categories: :56-95; simple lower-casing: :139-141).  The
product's tokenizer (cubert_amd/csrc/host/tokenization.cpp) has its own decoder, tables, decomposition and
reordering code; this file shares none of it.

Pinned by: every vector of the reference's test/cuBERT/tokenization_test.cpp (tests/golden/
tokenization_vectors.json), see tests/test_tokenizer.py.
"""
import unicodedata


def _category(cp):
    return unicodedata.category(chr(cp))


def is_whitespace(cp):
    """tokenization.cpp:56-61"""
    return cp in (0x20, 0x09, 0x0A, 0x0D) or _category(cp) == "Zs"


def is_control(cp):
    """tokenization.cpp:63-69: every C* category (not only Cc/Cf), except tab, newline, carriage return."""
    if cp in (0x09, 0x0A, 0x0D):
        return False
    return _category(cp)[0] == "C"


def is_punctuation(cp):
    """tokenization.cpp:71-82"""
    if 33 <= cp <= 47 or 58 <= cp <= 64 or 91 <= cp <= 96 or 123 <= cp <= 126:
        return True
    return _category(cp)[0] == "P"


def is_chinese_char(cp):
    """tokenization.cpp:97-114"""
    return (0x4E00 <= cp <= 0x9FFF or 0x3400 <= cp <= 0x4DBF or 0x20000 <= cp <= 0x2A6DF or
            0x2A700 <= cp <= 0x2B73F or 0x2B740 <= cp <= 0x2B81F or 0x2B820 <= cp <= 0x2CEAF or
            0xF900 <= cp <= 0xFAFF or 0x2F800 <= cp <= 0x2FA1F)


def simple_lower(cp):
    """utf8proc_tolower: the simple (one code point) lower-case mapping."""
    low = chr(cp).lower()
    if len(low) == 1:
        return ord(low)
    return 0x69 if cp == 0x130 else cp


def decode_prefix(raw):
    """Code points of the longest valid UTF-8 prefix of `raw` (the reference stops at a decode error,
    tokenization.cpp:133-137)."""
    try:
        return [ord(c) for c in raw.decode("utf8")]
    except UnicodeDecodeError as e:
        return [ord(c) for c in raw[:e.start].decode("utf8")]


def basic_tokenize(text, do_lower_case=True, max_length=1 << 30, tokens=None):
    """BasicTokenizer::tokenize, tokenization.cpp:116-183.  `text`: str or UTF-8 bytes."""
    raw = text.encode("utf8") if isinstance(text, str) else bytes(text)
    raw = raw.split(b"\0")[0]  # a C string ends at the first NUL
    cps = decode_prefix(raw)
    if do_lower_case:
        cps = [ord(c) for c in unicodedata.normalize("NFD", "".join(map(chr, cps)))]
    out = [] if tokens is None else tokens
    new_token = True
    for cp in cps:
        if do_lower_case:
            cp = simple_lower(cp)
        if cp == 0 or cp == 0xFFFD or is_control(cp):
            pass
        elif do_lower_case and _category(cp) == "Mn":
            pass
        elif is_whitespace(cp):
            new_token = True
        elif is_punctuation(cp) or is_chinese_char(cp):
            out.append(chr(cp))
            new_token = True
        else:
            if new_token:
                out.append(chr(cp))
                new_token = False
            else:
                out[-1] += chr(cp)
        if len(out) >= max_length:  # checked after the character: tokenization.cpp:175-178
            break
    return out


def wordpiece(token, vocab, unk_token="[UNK]", max_input_chars_per_word=200, tokens=None):
    """WordpieceTokenizer::tokenize, tokenization.cpp:186-216.  Lengths and cut points are BYTES of the UTF-8
    form, as there; a cut inside a character gives a candidate that is no vocabulary entry."""
    out = [] if tokens is None else tokens
    raw = token.encode("utf8") if isinstance(token, str) else bytes(token)
    if len(raw) > max_input_chars_per_word:
        out.append(unk_token)
        return out
    keep = len(out)
    start = 0
    while start < len(raw):
        found = None
        for end in range(len(raw), start, -1):
            cand = (b"##" if start > 0 else b"") + raw[start:end]
            try:
                key = cand.decode("utf8")
            except UnicodeDecodeError:
                continue
            if key in vocab:
                found = (key, end)
                break
        if found is None:
            del out[keep:]
            out.append(unk_token)
            return out
        out.append(found[0])
        start = found[1]
    return out


def load_vocab(lines):
    """load_vocab, tokenization.cpp:38-54: id = line number, lines stripped of the C locale's white space (not of
    Unicode separators such as U+2028, which the basic tokenizer keeps inside tokens); a repeated token keeps the
    last line number."""
    return {line.strip(" \t\n\v\f\r"): i for i, line in enumerate(lines)}


def full_tokenize(text, vocab, do_lower_case=True, max_length=1 << 30):
    """FullTokenizer::tokenize, tokenization.cpp:218-228."""
    out = []
    for token in basic_tokenize(text, do_lower_case, max_length):
        wordpiece(token, vocab, tokens=out)
        if len(out) >= max_length:
            break
    return out


def convert_single_example(vocab, max_seq_length, text_a, text_b=None, do_lower_case=True):
    """convert_single_example + _truncate_seq_pair, src/cuBERT.cpp:112-214 -> (ids, mask, segment ids)."""
    def token_id(t):
        return vocab.get(t, 0)

    a = full_tokenize(text_a, vocab, do_lower_case, max_seq_length)
    b = []
    if text_b is not None:
        b = full_tokenize(text_b, vocab, do_lower_case, max_seq_length)
        while len(a) + len(b) > max_seq_length - 3:
            if len(a) > len(b):
                a.pop()
            else:
                b.pop()
    else:
        a = a[:max_seq_length - 2]
    ids = [token_id("[CLS]")] + [token_id(t) for t in a] + [token_id("[SEP]")]
    seg = [0] * len(ids)
    if text_b is not None:
        ids += [token_id(t) for t in b] + [token_id("[SEP]")]
        seg += [1] * (len(b) + 1)
    n = len(ids)
    pad = max_seq_length - n
    return ids + [0] * pad, [1] * n + [0] * pad, seg + [0] * pad
