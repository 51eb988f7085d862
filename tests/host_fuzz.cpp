// Test driver, not part of the library: feeds damaged GraphDef files to Graph<T> and arbitrary byte strings to the
// tokenizer.  tests/test_host_sanitized.py compiles it together with csrc/host/Graph.cpp and tokenization.cpp under
// AddressSanitizer and UndefinedBehaviorSanitizer (host code only) and runs it: a read or write out of bounds, a
// leak, an overflow or any exception other than the documented std::invalid_argument ends it with a non-zero
// status.
//
//   host_fuzz <model.pb> <vocab.txt> <scratch file> <iterations> <seed>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

#include "Graph.h"
#include "tokenization.h"

namespace {

struct Rng {
    uint64_t s;
    uint64_t next() {
        s ^= s << 13, s ^= s >> 7, s ^= s << 17;
        return s;
    }
    size_t below(size_t n) { return n ? (size_t) (next() % n) : 0; }
};

std::vector<uint8_t> read_file(const char *path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) {
        fprintf(stderr, "host_fuzz: cannot read %s\n", path);
        exit(2);
    }
    return std::vector<uint8_t>((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
}

void write_file(const char *path, const std::vector<uint8_t> &bytes) {
    std::ofstream out(path, std::ios::binary | std::ios::trunc);
    out.write((const char *) bytes.data(), (std::streamsize) bytes.size());
    if (!out) {
        fprintf(stderr, "host_fuzz: cannot write %s\n", path);
        exit(2);
    }
}

struct Counts {
    size_t loaded = 0, refused = 0;
};

// Loads the file as both storage types; every tensor the loader returns must be readable over its whole stated
// size (the sanitizer checks the reads).  The only exception a damaged file may raise is std::invalid_argument.
template <typename T>
void load(const char *path, Counts *counts) {
    try {
        cuBERT::Graph<T> graph(path);
        double checksum = 0.0;
        for (const auto &kv : graph.var) {
            const size_t n = graph.size.at(kv.first);
            for (size_t i = 0; i < n; ++i) checksum += (double) (float) kv.second[i];
            (void) graph.shape.at(kv.first);
        }
        if (checksum == 12345.678) puts("");  // keeps the reads
        ++counts->loaded;
    } catch (const std::invalid_argument &) {
        ++counts->refused;
    }
}

void damage(std::vector<uint8_t> *bytes, Rng *rng) {
    const int edits = 1 + (int) rng->below(4);
    for (int e = 0; e < edits && !bytes->empty(); ++e) {
        const size_t at = rng->below(bytes->size());
        switch (rng->below(7)) {
            case 0: (*bytes)[at] ^= (uint8_t) (1u << rng->below(8)); break;
            case 1: (*bytes)[at] = 0xff; break;
            case 2: (*bytes)[at] = 0x80; break;
            case 3: (*bytes)[at] = (uint8_t) rng->next(); break;
            case 4: bytes->erase(bytes->begin() + (long) at, bytes->begin() + (long) std::min(bytes->size(), at + 1 + rng->below(16))); break;
            case 5: {  // a run of continuation bytes: an over-long or very large varint
                const size_t n = 1 + rng->below(11);
                bytes->insert(bytes->begin() + (long) at, n, (uint8_t) 0xff);
                break;
            }
            default: bytes->resize(at); break;
        }
    }
}

// Pieces a text is drawn from: ASCII, accented and combining characters, CJK, Hangul, a 4-byte character, control
// and format characters, white space of several kinds, and byte sequences that are not UTF-8.
const char *const kPieces[] = {"want", "ed", " ", "  ", "\t", "\n", ",", "!", "un", "running", "wa", "A", "Z",
                               "\xc3\xa9", "e\xcc\x81", "\xc3\x85", "\xe4\xb8\xad", "\xe6\x96\x87", "\xed\x95\x9c",
                               "\xf0\x9f\x98\x80", "\xe2\x80\x8b", "\xc2\xa0", "\xe3\x80\x80", "\x01", "\x7f",
                               "\xef\xbf\xbd", "\xcc\x81\xcc\xa7", "\xc7\x86", "\xe1\xba\x9e",
                               "\xff", "\xc3", "\xe4\xb8", "\xf0\x9f\x98", "\xc0\xaf", "\xed\xa0\x80", "\xf4\x90\x80\x80",
                               "\x80", "[UNK]", "[CLS]", "##ing", "#"};

std::string random_text(Rng *rng) {
    std::string s;
    const size_t pieces = rng->below(60);
    for (size_t i = 0; i < pieces; ++i) {
        if (rng->below(8) == 0) {
            const char c = (char) (1 + rng->below(255));  // never the terminator
            s.push_back(c);
        } else {
            s += kPieces[rng->below(sizeof(kPieces) / sizeof(kPieces[0]))];
        }
    }
    if (rng->below(16) == 0) s.append(300 + rng->below(200), 'a');  // a word past max_input_chars_per_word
    return s;
}

}  // namespace

int main(int argc, char **argv) {
    if (argc != 6) {
        fprintf(stderr, "usage: host_fuzz <model.pb> <vocab.txt> <scratch file> <iterations> <seed>\n");
        return 2;
    }
    const char *model = argv[1], *vocab_path = argv[2], *scratch = argv[3];
    const long iterations = atol(argv[4]);
    Rng rng{(uint64_t) atoll(argv[5]) * 0x9e3779b97f4a7c15ull + 1};
    std::cerr.setstate(std::ios::failbit);  // the loader's "model loaded from" lines; sanitizer reports do not pass here

    // ---- GraphDef loader ----
    const std::vector<uint8_t> good = read_file(model);
    Counts whole;
    load<float>(model, &whole);
    load<cuBERT::half>(model, &whole);
    if (whole.loaded != 2) {
        printf("the undamaged model file was refused\n");
        return 1;
    }
    Counts cut;
    for (size_t len = 0; len < good.size(); len += len < 256 ? 1 : 61) {  // every short prefix, then a stride
        write_file(scratch, std::vector<uint8_t>(good.begin(), good.begin() + (long) len));
        load<float>(scratch, &cut);
    }
    Counts damaged;
    for (long i = 0; i < iterations; ++i) {
        std::vector<uint8_t> bytes = good;
        damage(&bytes, &rng);
        write_file(scratch, bytes);
        if (i & 1) load<cuBERT::half>(scratch, &damaged);
        else load<float>(scratch, &damaged);
    }
    printf("graphdef: prefixes %zu loaded / %zu refused; damaged files %zu loaded / %zu refused\n", cut.loaded,
           cut.refused, damaged.loaded, damaged.refused);

    // ---- tokenizer ----
    cuBERT::FullTokenizer tokenizer(vocab_path, true), cased(vocab_path, false);
    size_t examples = 0, refused = 0;
    for (long i = 0; i < iterations * 4; ++i) {
        const std::string a = random_text(&rng), b = random_text(&rng);
        const bool pair = rng.below(2) == 1;
        const size_t seq = rng.below(8) == 0 ? rng.below(4) : 2 + rng.below(96);
        // exact-size output arrays: a write past max_seq_length is a heap overflow the sanitizer reports
        std::vector<int> ids(seq, -1);
        std::vector<int8_t> mask(seq, -1), segments(seq, -1);
        try {
            (i & 1 ? cased : tokenizer).convert_single_example(seq, a.c_str(), pair ? b.c_str() : nullptr, ids.data(),
                                                                mask.data(), segments.data());
        } catch (const std::invalid_argument &) {
            if (seq >= 3) {
                printf("convert_single_example refused seq_length %zu\n", seq);
                return 1;
            }
            ++refused;
            continue;
        }
        ++examples;
        size_t n = 0;
        while (n < seq && mask[n] == 1) ++n;
        bool ok = n >= (pair ? 3u : 2u);
        for (size_t t = 0; t < seq && ok; ++t) {
            ok = ids[t] >= 0 && (segments[t] == 0 || segments[t] == 1) && (t < n || (mask[t] == 0 && ids[t] == 0 && segments[t] == 0));
            if (t + 1 < n && segments[t] > segments[t + 1]) ok = false;  // segment ids never fall inside the example
        }
        if (!ok) {
            printf("convert_single_example wrote an inconsistent example (seq_length %zu)\n", seq);
            return 1;
        }
        std::vector<std::string> tokens;
        tokenizer.tokenize(a.c_str(), &tokens, 1 + rng.below(40));
        std::vector<uint64_t> token_ids(tokens.size());
        tokenizer.convert_tokens_to_ids(tokens, token_ids.data());
    }
    printf("tokenizer: %zu examples, %zu refused for a seq_length below the special tokens\n", examples, refused);
    puts("host_fuzz ok");
    return 0;
}
