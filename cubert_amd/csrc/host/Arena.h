// One device allocation carved into aligned tensors.  Used twice with the same
// layout code: a measuring pass (no memory yet, take() returns nullptr and only
// advances the cursor), allocate(), then the assigning pass.
#ifndef CUBERT_HOST_ARENA_H
#define CUBERT_HOST_ARENA_H

#include <cstddef>

#include "common.h"

namespace cuBERT {

class Arena {
public:
    Arena() = default;
    Arena(const Arena &) = delete;
    Arena &operator=(const Arena &) = delete;
    ~Arena() {
        if (base_ != nullptr) cuBERT::free(base_);
    }

    template <typename U>
    U *take(size_t count) {
        const size_t offset = (cursor_ + kAlign - 1) / kAlign * kAlign;
        cursor_ = offset + count * sizeof(U);
        return base_ == nullptr ? nullptr : reinterpret_cast<U *>(base_ + offset);
    }

    // Ends the measuring pass: allocates what was asked for and rewinds.  When the allocation fails (cuBERT::malloc
    // throws) the arena is empty and measuring again, so a later attempt asks for the same amount, not for more.
    void allocate() {
        size_ = cursor_;
        cursor_ = 0;
        base_ = static_cast<char *>(cuBERT::malloc(size_ == 0 ? kAlign : size_));
    }

    bool measuring() const { return base_ == nullptr; }
    size_t size() const { return size_; }

private:
    static constexpr size_t kAlign = 256;  // keeps every tensor 16-byte vector friendly and cache-line aligned
    char *base_ = nullptr;
    size_t cursor_ = 0;
    size_t size_ = 0;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_ARENA_H
