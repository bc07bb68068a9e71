// Host-only exercise of lg::StagingRing (logismos_amd/csrc/staging_ring.hpp) with a
// simulated stream: copies run only when the test says so, as a busy device would run them.
// Exit status 0 = every check passed.
#include "staging_ring.hpp"

#include <cstdio>
#include <deque>
#include <vector>

struct FakeStream {
    struct Copy {
        const int32_t* src;
        int count;
        int dst_off;
        int fence_after;  // slot whose fence is recorded right behind this copy
    };
    std::deque<Copy> queue;
    std::vector<int32_t> device = std::vector<int32_t>(64, -1);
    std::vector<int> reached;  // fences reached, per slot
    int waits = 0;
    void run_one() {
        Copy c = queue.front();
        queue.pop_front();
        for (int i = 0; i < c.count; ++i) device[(size_t)(c.dst_off + i)] = c.src[i];
        if (c.fence_after >= 0) reached[(size_t)c.fence_after]++;
    }
};

struct FakeFence {
    FakeStream* st = nullptr;
    std::vector<int>* recorded = nullptr;
    void record(int slot, FakeStream*) {
        st->queue.back().fence_after = slot;
        (*recorded)[(size_t)slot]++;
    }
    void wait(int slot) {
        st->waits++;
        // "block": the device makes progress until this slot's latest fence is reached
        while (st->reached[(size_t)slot] < (*recorded)[(size_t)slot]) st->run_one();
    }
};

#define CHECK(c)                                                   \
    do {                                                           \
        if (!(c)) {                                                \
            std::printf("FAILED line %d: %s\n", __LINE__, #c);     \
            return 1;                                              \
        }                                                          \
    } while (0)

int main() {
    const int slots = 3, elems = 4;
    std::vector<int32_t> pinned((size_t)slots * elems, 0);
    FakeStream st;
    st.reached.assign(slots, 0);
    std::vector<int> recorded(slots, 0);
    lg::StagingRing<FakeFence, FakeStream*> ring;
    ring.init(pinned.data(), slots, elems, FakeFence{&st, &recorded});

    // the bookkeeping row of one sequence slot, rewritten by successive owners while NO copy
    // has run yet: each queued copy must still deliver what the row held when it was queued
    int32_t row[4] = {10, 11, 12, 13};
    auto update = [&](int dst_off) {
        int32_t* staged = nullptr;
        const int slot = ring.stage(row, 4, &staged);
        st.queue.push_back({staged, 4, dst_off, -1});
        ring.queued(slot, &st);
    };
    update(0);
    row[0] = 20; row[1] = 21; row[2] = 22; row[3] = 23;   // slot closed, reopened, regrown
    update(4);
    row[0] = 30; row[1] = 31; row[2] = 32; row[3] = 33;
    update(8);
    CHECK(st.queue.size() == 3 && st.waits == 0);          // three slots: nothing had to wait
    // a fourth update needs slot 0 again: the ring must wait for (run) the first copy, and
    // only that one, before it overwrites the slot
    row[0] = 40; row[1] = 41; row[2] = 42; row[3] = 43;
    update(12);
    CHECK(st.waits == 1);
    CHECK(st.device[0] == 10 && st.device[3] == 13);       // first copy ran with ITS contents
    CHECK(st.queue.size() == 3);                           // the others are still queued
    while (!st.queue.empty()) st.run_one();
    const int32_t want[16] = {10, 11, 12, 13, 20, 21, 22, 23, 30, 31, 32, 33, 40, 41, 42, 43};
    for (int i = 0; i < 16; ++i) CHECK(st.device[(size_t)i] == want[i]);
    // fences already reached are not waited for again ...
    const int waits_before = st.waits;
    update(16);
    update(20);
    update(24);
    CHECK(st.waits == waits_before + 3);   // each slot was armed once more: one (instant) wait
    // ... and drain() leaves nothing queued
    ring.drain();
    CHECK(st.queue.empty());
    CHECK(st.device[16] == 40 && st.device[24] == 40);
    std::printf("staging ring ok\n");
    return 0;
}
