// A ring of host staging slots for small asynchronous host-to-device updates.
//
// An asynchronous copy reads its host source when the copy RUNS, not when it is queued.
// Bookkeeping memory that the host keeps rewriting (a block-table row whose sequence slot is
// closed, reopened and grown again) is therefore no safe source: a queued copy of the old
// owner's entries would carry the new owner's.  Every update is first copied into a slot of
// this ring; a slot is handed out again only after the fence recorded behind its copy reports
// that the copy has run (the ring waits for it if it has to).
//
// The fence is a policy so that the hand-out rule can be exercised on the host without a
// device: `Fence` provides  void record(int slot, Stream)  -- mark "everything queued on the
// stream so far", called right after the slot's copy was queued;  void wait(int slot)  --
// block until that mark is reached.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <vector>

namespace lg {

template <class Fence, class Stream>
class StagingRing {
public:
    StagingRing() = default;
    // `memory`: slots * slot_elems int32 of (pinned) host memory owned by the caller
    void init(int32_t* memory, int slots, int slot_elems, Fence fence) {
        mem_ = memory;
        slots_ = slots;
        slot_elems_ = slot_elems;
        fence_ = fence;
        armed_.assign((size_t)slots, 0);
        next_ = 0;
    }
    int slot_elems() const { return slot_elems_; }
    int slots() const { return slots_; }

    // Copies `count` (<= slot_elems) entries into the next slot, waiting first for the copy
    // that last used that slot.  Returns the slot index; `*staged` points at the slot.
    int stage(const int32_t* src, int count, int32_t** staged) {
        const int s = next_;
        next_ = (next_ + 1) % slots_;
        if (armed_[(size_t)s]) {
            fence_.wait(s);
            armed_[(size_t)s] = 0;
        }
        int32_t* dst = mem_ + (size_t)s * slot_elems_;
        std::memcpy(dst, src, sizeof(int32_t) * (size_t)count);
        *staged = dst;
        return s;
    }
    // To be called right after the copy out of `slot` has been queued on `stream`.
    void queued(int slot, Stream stream) {
        fence_.record(slot, stream);
        armed_[(size_t)slot] = 1;
    }
    // Blocks until every queued copy has run (destroy, reset of the owner).
    void drain() {
        for (int s = 0; s < slots_; ++s)
            if (armed_[(size_t)s]) {
                fence_.wait(s);
                armed_[(size_t)s] = 0;
            }
    }

private:
    int32_t* mem_ = nullptr;
    int slots_ = 0, slot_elems_ = 0, next_ = 0;
    Fence fence_{};
    std::vector<uint8_t> armed_;
};

}  // namespace lg
