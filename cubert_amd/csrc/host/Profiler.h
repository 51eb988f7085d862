// Optional per-kernel timing of a forward pass with stream events: a pair of
// events is recorded around each launch of the kinds that are switched on, and
// read back after the stream has been synchronised.  Off by default (no events
// are recorded then).  The reference has no counterpart.
#ifndef CUBERT_HOST_PROFILER_H
#define CUBERT_HOST_PROFILER_H

#include <utility>
#include <vector>

#include "common.h"

namespace cuBERT {

class Profiler {
public:
    enum Kind {
        kEmbedLayerNorm = 0,
        kBiasResLayerNorm = 1,
        kBiasGelu = 2,
        kMaskScaleSoftmax = 3,
        kBiasTanh = 4,
        kMeanPool = 5,
        kRowSoftmax = 6,
        kDenseGemm = 7,
        kAttentionGemm = 8,
        kAttentionFused = 9,
        kClassifierHead = 10,
        kDenseSplit = 11,  // fp32 rows written as two-term fp16 rows ahead of a Dense GEMM
        // The Dense GEMMs one by one: a Dense launch is timed under its own kind when that kind is on, under
        // kDenseGemm otherwise (so a caller sees either the sum or the parts, never the same launch twice).
        kDenseQkv = 12,              // Q | K | V projection, [hidden] -> [3 * hidden]
        kDenseAttentionOutput = 13,  // attention output, [hidden] -> [hidden]
        kDenseIntermediate = 14,     // feed-forward up, [hidden] -> [intermediate]
        kDenseOutput = 15,           // feed-forward down, [intermediate] -> [hidden]
        kDensePooler = 16,           // BertPooler, [hidden] -> [hidden] on the first token of every sequence
        kKinds = 17
    };

    // The kind a Dense launch is timed under: its own when that is on, else the aggregate.
    Kind dense_kind(Kind detail) const { return on(detail) ? detail : kDenseGemm; }

    ~Profiler() {
        for (auto &e : pool) {
            cubert_event_destroy(e.first);
            cubert_event_destroy(e.second);
        }
    }

    // Bit k of `kinds` switches timing of Kind k on; 0 switches everything off.
    void enable(unsigned kinds) {
        mask = kinds;
        if (mask != 0) grow(1024);
    }

    bool on(Kind k) const { return (mask >> k) & 1u; }

    // The layer kernels (kinds 0..6) and the one-launch attention kernel are one launch each: the launch itself
    // carries the event pair and the elapsed time is the kernel's execution time.  GEMM kinds may be several
    // library launches, so they are bracketed by marker events (which adds the gaps between launches).
    static bool single_launch(Kind k) { return k < kDenseGemm || k == kAttentionFused || k == kClassifierHead; }

    void begin(Kind k, void *stream) {
        if (!on(k)) return;
        if (used == pool.size()) grow(pool.size() + 1024);
        if (single_launch(k)) {
            CUBERT_CHECK(cubert_time_next_launch(pool[used].first, pool[used].second));
        } else {
            CUBERT_CHECK(cubert_event_record(pool[used].first, stream));
        }
    }

    // The entry point under a single-launch bracket declined and launched nothing: the pair goes back unused.
    void cancel(Kind k) {
        if (!on(k) || !single_launch(k)) return;
        CUBERT_CHECK(cubert_time_next_launch(nullptr, nullptr));
        cancelled = true;
    }

    void end(Kind k, void *stream) {
        if (!on(k)) return;
        if (cancelled) {
            cancelled = false;
            return;
        }
        if (!single_launch(k)) CUBERT_CHECK(cubert_event_record(pool[used].second, stream));
        kinds_used.push_back(k);
        ++used;
    }

    // Adds the elapsed time of every pair recorded since the last call to total_ms[kind] / count[kind]
    // and forgets them.  The stream must have been synchronised.
    void collect(double *total_ms, int *count) {
        for (size_t i = 0; i < used; ++i) {
            float ms = 0.f;
            CUBERT_CHECK(cubert_event_elapsed_ms(pool[i].first, pool[i].second, &ms));
            total_ms[kinds_used[i]] += ms;
            count[kinds_used[i]] += 1;
        }
        used = 0;
        kinds_used.clear();
    }

private:
    void grow(size_t n) {
        while (pool.size() < n) {
            void *a = cubert_event_create(), *b = cubert_event_create();
            if (!a || !b) {
                fprintf(stderr, "cuBERT: could not create timing events\n");
                exit(EXIT_FAILURE);
            }
            pool.emplace_back(a, b);
        }
    }

    unsigned mask = 0;
    bool cancelled = false;
    size_t used = 0;
    std::vector<std::pair<void *, void *>> pool;
    std::vector<Kind> kinds_used;
};

// RAII bracket around one launch; does nothing when `p` is null or the kind is off.
class Timed {
public:
    Timed(Profiler *p, Profiler::Kind k, void *stream) : p(p), k(k), stream(stream) {
        if (p) p->begin(k, stream);
    }
    ~Timed() {
        if (p) p->end(k, stream);
    }
    // nothing was launched inside this bracket
    void cancel() {
        if (p) p->cancel(k);
    }

private:
    Profiler *p;
    Profiler::Kind k;
    void *stream;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_PROFILER_H
