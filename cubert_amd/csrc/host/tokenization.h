// BERT text front end: basic tokenizer (clean-up, lower-casing with accent stripping, punctuation and CJK
// splitting), greedy WordPiece, vocabulary lookup.  Class and function names follow the reference
// (src/cuBERT/tokenization.h:10-152); the Unicode properties come from tables generated beside this file
// (gen_unicode_tables.py) instead of utf8proc.
#ifndef CUBERT_HOST_TOKENIZATION_H
#define CUBERT_HOST_TOKENIZATION_H

#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace cuBERT {

// One token per line, id = line number (reference: tokenization.cpp:38-54).  Lines are stripped of
// surrounding white space; a repeated token keeps its last line number.  Throws std::invalid_argument
// when the file cannot be opened.
void load_vocab(const char *vocab_file, std::unordered_map<std::string, uint64_t> *vocab);

// Character classes of the basic tokenizer (reference: tokenization.cpp:56-95).
bool _is_whitespace(int cp);   // space, \t, \n, \r and category Zs
bool _is_control(int cp);      // any category C* except \t, \n, \r
bool _is_punctuation(int cp);  // ASCII non-alphanumerics and category P*

namespace unicode {
// Decodes strictly (no overlong forms, surrogates or values above U+10FFFF).  Returns the number of bytes
// consumed, or -1 at an invalid sequence.
int decode_utf8(const unsigned char *s, size_t n, uint32_t *cp);
void append_utf8(uint32_t cp, std::string *out);
uint32_t to_lower(uint32_t cp);  // simple lower-case mapping
// Canonical decomposition with canonical reordering (NFD) of a code point sequence.
void nfd(const std::vector<uint32_t> &in, std::vector<uint32_t> *out);
const char *version();
}  // namespace unicode

class BasicTokenizer {
public:
    explicit BasicTokenizer(bool do_lower_case = true) : do_lower_case(do_lower_case) {}
    BasicTokenizer(const BasicTokenizer &) = delete;

    // Appends the tokens of `text` to `output_tokens`; stops once it holds max_length tokens.
    // Text after an invalid UTF-8 sequence is dropped (with a message on stderr), as in the reference.
    void tokenize(const char *text, std::vector<std::string> *output_tokens, size_t max_length) const;

private:
    const bool do_lower_case;
};

class WordpieceTokenizer {
public:
    explicit WordpieceTokenizer(const std::unordered_map<std::string, uint64_t> *vocab,
                                std::string unk_token = "[UNK]", int max_input_chars_per_word = 200);
    WordpieceTokenizer(const WordpieceTokenizer &) = delete;

    // Greedy longest-match-first split of one basic token into word pieces ("unaffable" -> un ##aff
    // ##able); a token with an unmatched remainder, or longer than max_input_chars_per_word bytes,
    // becomes unk_token.  Lengths are bytes, like the reference (tokenization.cpp:186-216).
    void tokenize(const std::string &token, std::vector<std::string> *output_tokens) const;

private:
    const std::unordered_map<std::string, uint64_t> *vocab;
    const std::string unk_token;
    const size_t max_input_chars_per_word;
};

class FullTokenizer {
public:
    explicit FullTokenizer(const char *vocab_file, bool do_lower_case = true);
    FullTokenizer(const FullTokenizer &) = delete;

    void tokenize(const char *text, std::vector<std::string> *output_tokens, size_t max_length) const;

    // The WordPiece step alone, on one basic token.
    void wordpiece(const std::string &token, std::vector<std::string> *output_tokens) const {
        wordpiece_tokenizer.tokenize(token, output_tokens);
    }

    // Id of a token; a token that is not in the vocabulary gives 0 and a message on stderr.
    uint64_t convert_token_to_id(const std::string &token) const;
    void convert_tokens_to_ids(const std::vector<std::string> &tokens, uint64_t *ids) const;

    // One example -> [CLS] a [SEP] (b [SEP]) ids, mask and segment ids, zero padded to max_seq_length
    // (reference: convert_single_example and _truncate_seq_pair, src/cuBERT.cpp:112-214).  text_b may be null.
    void convert_single_example(size_t max_seq_length, const char *text_a, const char *text_b, int *input_ids,
                                int8_t *input_mask, int8_t *segment_ids) const;

private:
    std::unordered_map<std::string, uint64_t> vocab;
    BasicTokenizer basic_tokenizer;
    WordpieceTokenizer wordpiece_tokenizer;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_TOKENIZATION_H
