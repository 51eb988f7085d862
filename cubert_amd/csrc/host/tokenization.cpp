#include "tokenization.h"

#include <algorithm>
#include <cctype>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>

namespace cuBERT {

namespace {

struct ClassRange {
    uint32_t first, last;
    uint8_t value;
};
struct CodePointPair {
    uint32_t from, to;
};
struct DecompositionEntry {
    uint32_t cp;
    uint16_t offset, length;
};

#include "unicode_tables.inc"

enum CharClass { kOther = 0, kControl = 1, kNonspacingMark = 2, kSpaceSeparator = 3, kPunctuation = 4 };

template <size_t N>
int range_value(const ClassRange (&table)[N], uint32_t cp) {
    size_t lo = 0, hi = N;
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (cp > table[mid].last) lo = mid + 1;
        else hi = mid;
    }
    return lo < N && cp >= table[lo].first ? table[lo].value : 0;
}

int char_class(int cp) {
    if (cp < 0 || cp > 0x10FFFF) return kControl;  // not a code point: treated as unassigned
    return range_value(kClassRanges, (uint32_t) cp);
}

int combining_class(uint32_t cp) { return range_value(kCombiningRanges, cp); }

// Hangul syllable arithmetic (Unicode chapter 3.12)
constexpr uint32_t kSBase = 0xAC00, kLBase = 0x1100, kVBase = 0x1161, kTBase = 0x11A7;
constexpr uint32_t kVCount = 21, kTCount = 28, kSCount = 19 * kVCount * kTCount;

void decompose(uint32_t cp, std::vector<uint32_t> *out) {
    if (cp >= kSBase && cp < kSBase + kSCount) {
        const uint32_t s = cp - kSBase;
        out->push_back(kLBase + s / (kVCount * kTCount));
        out->push_back(kVBase + (s % (kVCount * kTCount)) / kTCount);
        if (s % kTCount) out->push_back(kTBase + s % kTCount);
        return;
    }
    const DecompositionEntry *end = kDecomposition + sizeof kDecomposition / sizeof kDecomposition[0];
    const DecompositionEntry *it = std::lower_bound(
            kDecomposition, end, cp, [](const DecompositionEntry &e, uint32_t v) { return e.cp < v; });
    if (it != end && it->cp == cp) {
        out->insert(out->end(), kDecompositionPool + it->offset, kDecompositionPool + it->offset + it->length);
    } else {
        out->push_back(cp);
    }
}

bool is_chinese_char(uint32_t cp) {
    // the CJK ideograph blocks of the reference (tokenization.cpp:97-114)
    return (cp >= 0x4E00 && cp <= 0x9FFF) || (cp >= 0x3400 && cp <= 0x4DBF) || (cp >= 0x20000 && cp <= 0x2A6DF) ||
           (cp >= 0x2A700 && cp <= 0x2B73F) || (cp >= 0x2B740 && cp <= 0x2B81F) || (cp >= 0x2B820 && cp <= 0x2CEAF) ||
           (cp >= 0xF900 && cp <= 0xFAFF) || (cp >= 0x2F800 && cp <= 0x2FA1F);
}

bool is_whitespace_class(int cp, int cls) {
    return cp == ' ' || cp == '\t' || cp == '\n' || cp == '\r' || cls == kSpaceSeparator;
}

bool is_control_class(int cp, int cls) {
    if (cp == '\t' || cp == '\n' || cp == '\r') return false;  // counted as white space
    return cls == kControl;
}

bool is_punctuation_class(int cp, int cls) {
    // all ASCII that is not a letter, digit or space counts, also "^", "$", "`" which Unicode calls symbols
    if ((cp >= 33 && cp <= 47) || (cp >= 58 && cp <= 64) || (cp >= 91 && cp <= 96) || (cp >= 123 && cp <= 126)) return true;
    return cls == kPunctuation;
}

std::string strip(const std::string &s) {
    size_t a = 0, b = s.size();
    while (a < b && std::isspace((unsigned char) s[a])) ++a;
    while (b > a && std::isspace((unsigned char) s[b - 1])) --b;
    return s.substr(a, b - a);
}

}  // namespace

bool _is_whitespace(int cp) { return is_whitespace_class(cp, char_class(cp)); }
bool _is_control(int cp) { return is_control_class(cp, char_class(cp)); }
bool _is_punctuation(int cp) { return is_punctuation_class(cp, char_class(cp)); }

namespace unicode {

const char *version() { return kUnicodeVersion; }

int decode_utf8(const unsigned char *s, size_t n, uint32_t *cp) {
    if (n == 0) return -1;
    const unsigned c0 = s[0];
    if (c0 < 0x80) {
        *cp = c0;
        return 1;
    }
    int len;
    uint32_t v, min;
    if (c0 >= 0xC2 && c0 <= 0xDF) { len = 2; v = c0 & 0x1F; min = 0x80; }
    else if (c0 >= 0xE0 && c0 <= 0xEF) { len = 3; v = c0 & 0x0F; min = 0x800; }
    else if (c0 >= 0xF0 && c0 <= 0xF4) { len = 4; v = c0 & 0x07; min = 0x10000; }
    else return -1;
    if ((size_t) len > n) return -1;
    for (int i = 1; i < len; ++i) {
        if ((s[i] & 0xC0) != 0x80) return -1;
        v = (v << 6) | (s[i] & 0x3F);
    }
    if (v < min || v > 0x10FFFF || (v >= 0xD800 && v <= 0xDFFF)) return -1;
    *cp = v;
    return len;
}

void append_utf8(uint32_t cp, std::string *out) {
    if (cp < 0x80) {
        out->push_back((char) cp);
    } else if (cp < 0x800) {
        out->push_back((char) (0xC0 | (cp >> 6)));
        out->push_back((char) (0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
        out->push_back((char) (0xE0 | (cp >> 12)));
        out->push_back((char) (0x80 | ((cp >> 6) & 0x3F)));
        out->push_back((char) (0x80 | (cp & 0x3F)));
    } else {
        out->push_back((char) (0xF0 | (cp >> 18)));
        out->push_back((char) (0x80 | ((cp >> 12) & 0x3F)));
        out->push_back((char) (0x80 | ((cp >> 6) & 0x3F)));
        out->push_back((char) (0x80 | (cp & 0x3F)));
    }
}

uint32_t to_lower(uint32_t cp) {
    if (cp < 0x80) return cp >= 'A' && cp <= 'Z' ? cp + 32 : cp;
    const CodePointPair *end = kLower + sizeof kLower / sizeof kLower[0];
    const CodePointPair *it =
            std::lower_bound(kLower, end, cp, [](const CodePointPair &e, uint32_t v) { return e.from < v; });
    return it != end && it->from == cp ? it->to : cp;
}

void nfd(const std::vector<uint32_t> &in, std::vector<uint32_t> *out) {
    out->clear();
    out->reserve(in.size() + in.size() / 4);
    for (uint32_t cp : in) {
        if (cp < 0xC0) out->push_back(cp);  // nothing below U+00C0 decomposes
        else decompose(cp, out);
    }
    // canonical ordering: within every run of marks (combining class != 0), stable sort by class
    size_t i = 0;
    const size_t n = out->size();
    while (i < n) {
        if ((*out)[i] < 0x300 || combining_class((*out)[i]) == 0) {
            ++i;
            continue;
        }
        size_t j = i;
        while (j < n && (*out)[j] >= 0x300 && combining_class((*out)[j]) != 0) ++j;
        if (j - i > 1) {
            std::stable_sort(out->begin() + i, out->begin() + j,
                             [](uint32_t a, uint32_t b) { return combining_class(a) < combining_class(b); });
        }
        i = j;
    }
}

}  // namespace unicode

void load_vocab(const char *vocab_file, std::unordered_map<std::string, uint64_t> *vocab) {
    std::ifstream file(vocab_file);
    if (!file) throw std::invalid_argument("Unable to open vocab file");
    uint64_t index = 0;
    std::string line;
    while (std::getline(file, line)) (*vocab)[strip(line)] = index++;
}

void BasicTokenizer::tokenize(const char *text, std::vector<std::string> *output_tokens, size_t max_length) const {
    // decode once; with lower-casing the whole text is decomposed first so that accents become separate
    // marks (category Mn), which are then dropped
    std::vector<uint32_t> cps;
    const unsigned char *s = (const unsigned char *) text;
    size_t left = std::strlen(text);
    while (left > 0) {
        uint32_t cp;
        const int len = unicode::decode_utf8(s, left, &cp);
        if (len < 0) {
            std::cerr << "UTF-8 decode error: " << text << std::endl;
            break;
        }
        cps.push_back(cp);
        s += len;
        left -= (size_t) len;
    }
    std::vector<uint32_t> decomposed;
    if (do_lower_case) {
        unicode::nfd(cps, &decomposed);
        cps.swap(decomposed);
    }

    bool new_token = true;
    for (uint32_t raw : cps) {
        const uint32_t cp = do_lower_case ? unicode::to_lower(raw) : raw;
        const int cls = char_class((int) cp);
        if (cp == 0 || cp == 0xFFFD || is_control_class((int) cp, cls)) {
            // dropped
        } else if (do_lower_case && cls == kNonspacingMark) {
            // an accent split off by the decomposition: dropped
        } else if (is_whitespace_class((int) cp, cls)) {
            new_token = true;
        } else if (is_punctuation_class((int) cp, cls) || is_chinese_char(cp)) {
            output_tokens->emplace_back();
            unicode::append_utf8(cp, &output_tokens->back());
            new_token = true;
        } else {
            if (new_token) output_tokens->emplace_back();
            unicode::append_utf8(cp, &output_tokens->back());
            new_token = false;
        }
        // The check comes after the character, as in the reference (tokenization.cpp:175-178): the token that
        // reaches max_length is cut after its first character.
        if (output_tokens->size() >= max_length) break;
    }
}

WordpieceTokenizer::WordpieceTokenizer(const std::unordered_map<std::string, uint64_t> *vocab, std::string unk_token,
                                       int max_input_chars_per_word)
        : vocab(vocab), unk_token(std::move(unk_token)),
          max_input_chars_per_word((size_t) std::max(0, max_input_chars_per_word)) {}

void WordpieceTokenizer::tokenize(const std::string &token, std::vector<std::string> *output_tokens) const {
    if (token.size() > max_input_chars_per_word) {
        output_tokens->push_back(unk_token);
        return;
    }
    const size_t first_piece = output_tokens->size();
    std::string candidate;
    for (size_t start = 0; start < token.size();) {
        size_t end = token.size();
        bool found = false;
        for (; end > start; --end) {
            candidate.assign(start > 0 ? "##" : "");
            candidate.append(token, start, end - start);
            if (vocab->count(candidate)) {
                found = true;
                break;
            }
        }
        if (!found) {
            output_tokens->resize(first_piece);
            output_tokens->push_back(unk_token);
            return;
        }
        output_tokens->push_back(candidate);
        start = end;
    }
}

FullTokenizer::FullTokenizer(const char *vocab_file, bool do_lower_case)
        : basic_tokenizer(do_lower_case), wordpiece_tokenizer(&vocab) {
    load_vocab(vocab_file, &vocab);
}

void FullTokenizer::tokenize(const char *text, std::vector<std::string> *output_tokens, size_t max_length) const {
    std::vector<std::string> tokens;
    tokens.reserve(max_length);
    basic_tokenizer.tokenize(text, &tokens, max_length);
    for (const std::string &token : tokens) {
        wordpiece_tokenizer.tokenize(token, output_tokens);
        if (output_tokens->size() >= max_length) break;
    }
}

uint64_t FullTokenizer::convert_token_to_id(const std::string &token) const {
    auto it = vocab.find(token);
    if (it == vocab.end()) {
        std::cerr << "vocab missing key: " << token << std::endl;
        return 0;
    }
    return it->second;
}

void FullTokenizer::convert_tokens_to_ids(const std::vector<std::string> &tokens, uint64_t *ids) const {
    for (size_t i = 0; i < tokens.size(); ++i) ids[i] = convert_token_to_id(tokens[i]);
}

void FullTokenizer::convert_single_example(size_t max_seq_length, const char *text_a, const char *text_b,
                                           int *input_ids, int8_t *input_mask, int8_t *segment_ids) const {
    const size_t specials = text_b ? 3 : 2;  // [CLS], [SEP] (, [SEP])
    if (max_seq_length < specials) throw std::invalid_argument("seq_length too short for [CLS] and [SEP]");
    std::vector<std::string> a, b;
    tokenize(text_a, &a, max_seq_length);
    if (text_b) {
        tokenize(text_b, &b, max_seq_length);
        // drop tokens from the end of whichever sequence is longer (b on a tie) until the pair fits
        while (a.size() + b.size() > max_seq_length - specials) {
            if (a.size() > b.size()) a.pop_back();
            else b.pop_back();
        }
    } else if (a.size() > max_seq_length - specials) {
        a.resize(max_seq_length - specials);
    }

    size_t n = 0;
    auto put = [&](const std::string &token, int8_t segment) {
        input_ids[n] = (int) convert_token_to_id(token);
        segment_ids[n] = segment;
        ++n;
    };
    put("[CLS]", 0);
    for (const std::string &t : a) put(t, 0);
    put("[SEP]", 0);
    if (text_b) {
        for (const std::string &t : b) put(t, 1);
        put("[SEP]", 1);
    }
    std::fill_n(input_mask, n, (int8_t) 1);
    std::fill_n(input_ids + n, max_seq_length - n, 0);
    std::fill_n(input_mask + n, max_seq_length - n, (int8_t) 0);
    std::fill_n(segment_ids + n, max_seq_length - n, (int8_t) 0);
}

}  // namespace cuBERT
