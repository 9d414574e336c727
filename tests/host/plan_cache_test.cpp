// CPU test of the plan cache's slot state machine (torchopt_amd/csrc/plan_cache.hpp) with a fake
// backend that models what the device would be doing: launches in flight per stream, events
// behind them, and memory that must be neither freed nor rewritten from another stream while a
// launch may still read it.  Prints "ok" and exits 0, or names the first broken expectation.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <thread>
#include <vector>

#include "plan_cache.hpp"

#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            std::exit(1);                                                   \
        }                                                                   \
    } while (0)

namespace {

struct Device {  // shared by every copy of the backend
    std::map<void *, size_t> live;                 // allocated blocks
    std::map<void *, std::set<void *>> readers;    // block -> streams with launches in flight
    std::map<void *, uint64_t> enqueued, finished; // per stream: work items so far
    size_t allocs = 0, blocking_frees = 0, freed_while_read = 0;
    uintptr_t next = 0x1000;
};

struct FakeBackend {
    struct Event {
        void *stream = nullptr;
        uint64_t at = 0;
    };
    Device *dev;
    bool fail_alloc = false;
    void *alloc(size_t bytes) {
        if (fail_alloc) return nullptr;
        void *p = reinterpret_cast<void *>(dev->next);
        dev->next += (bytes + 0xfff) & ~(uintptr_t)0xfff;
        dev->live[p] = bytes;
        ++dev->allocs;
        return p;
    }
    void free_blocking(int, void *p) {  // the device drains first
        for (auto &s : dev->enqueued) dev->finished[s.first] = s.second;
        dev->readers.clear();
        EXPECT(dev->live.count(p) == 1);
        dev->live.erase(p);
        ++dev->blocking_frees;
    }
    bool record(void *stream, Event *out) {
        *out = Event{stream, dev->enqueued[stream]};
        return true;
    }
    bool done(const Event &e) { return dev->finished[e.stream] >= e.at; }
    void drop(Event &) {}
};

struct Memo {
    int tag = 0;
};
using Cache = toa::PlanCache<FakeBackend, Memo>;
using Bytes = Cache::Bytes;

Bytes key_of(int k, size_t len = 8) { return Bytes(len, (unsigned char)k); }

// what the library does with a slot: (re)write on the stream if fresh, then a launch that reads it
void serve(Cache &cache, Device &dev, Cache::Slot *slot, bool fresh, void *stream, const Bytes &key) {
    EXPECT(slot->stream == stream);
    if (fresh) {
        // a rewrite is ordered behind earlier readers only on the slot's own stream
        for (void *reader : dev.readers[slot->mem]) EXPECT(reader == stream);
        ++dev.enqueued[stream];
        cache.commit(slot, Bytes(key));
    }
    ++dev.enqueued[stream];
    dev.readers[slot->mem].insert(stream);
}

void drain(Device &dev, void *stream) {
    dev.finished[stream] = dev.enqueued[stream];
    for (auto &r : dev.readers) r.second.erase(stream);
}

void *S(int i) { return reinterpret_cast<void *>((uintptr_t)0x100 * (i + 1)); }

void test_hit_and_lru() {
    Device dev;
    Cache cache(FakeBackend{&dev});
    bool fresh = false;
    const int P = (int)toa::kPlanSlotsPerStream;
    std::vector<void *> mem;
    for (int k = 0; k < P; ++k) {
        Cache::Slot *s = cache.acquire(0, S(0), key_of(k), 1000, &fresh);
        EXPECT(s != nullptr && fresh);
        serve(cache, dev, s, fresh, S(0), key_of(k));
        mem.push_back(s->mem);
    }
    EXPECT((int)cache.slots() == P && (int)dev.allocs == P);
    // hits: same memory, nothing to write
    for (int k = 0; k < P; ++k) {
        Cache::Slot *s = cache.acquire(0, S(0), key_of(k), 1000, &fresh);
        EXPECT(s != nullptr && !fresh && s->mem == mem[k]);
    }
    // touch 0, then one list more than the stream may keep evicts the least recently used: list 1
    cache.acquire(0, S(0), key_of(0), 1000, &fresh);
    Cache::Slot *s = cache.acquire(0, S(0), key_of(1000), 1000, &fresh);
    EXPECT(s != nullptr && fresh && s->mem == mem[1]);  // rewritten in place, same stream
    serve(cache, dev, s, fresh, S(0), key_of(1000));
    EXPECT((int)cache.slots() == P && (int)dev.allocs == P && dev.blocking_frees == 0);
    s = cache.acquire(0, S(0), key_of(1), 1000, &fresh);
    EXPECT(fresh);  // list 1 is gone
    // another stream gets slots of its own
    s = cache.acquire(0, S(1), key_of(0), 1000, &fresh);
    EXPECT(s != nullptr && fresh && (int)cache.slots() == P + 1);
    // and so does another device
    s = cache.acquire(1, S(0), key_of(0), 1000, &fresh);
    EXPECT(s != nullptr && fresh && (int)cache.slots() == P + 2);
}

void test_grow_parks_memory_until_its_readers_are_done() {
    Device dev;
    Cache cache(FakeBackend{&dev});
    bool fresh = false;
    for (int k = 0; k < (int)toa::kPlanSlotsPerStream; ++k) {
        Cache::Slot *s = cache.acquire(0, S(0), key_of(k), 1000, &fresh);
        serve(cache, dev, s, fresh, S(0), key_of(k));
    }
    const size_t live_before = dev.live.size();
    // one list more, and a longer one: the evicted slot's memory is too small and still being read
    Cache::Slot *s = cache.acquire(0, S(0), key_of(1007), 100000, &fresh);
    EXPECT(s != nullptr && fresh && s->capacity >= 100000);
    EXPECT(dev.blocking_frees == 0);                 // nothing waited, nothing freed
    EXPECT(dev.live.size() == live_before + 1);      // the old block is parked, not gone
    EXPECT(cache.parked() == 1);
    serve(cache, dev, s, fresh, S(0), key_of(1007));
    // while the stream has not drained the parked block is not handed out again
    s = cache.acquire(0, S(0), key_of(1008), 100000, &fresh);
    EXPECT(s != nullptr && fresh && cache.parked() == 2 && dev.blocking_frees == 0);
    serve(cache, dev, s, fresh, S(0), key_of(1008));
    drain(dev, S(0));
    // now a small new list may reuse a parked block instead of allocating
    const size_t allocs = dev.allocs;
    s = cache.acquire(0, S(1), key_of(1), 500, &fresh);
    EXPECT(s != nullptr && fresh && dev.allocs == allocs && cache.parked() == 1);
    EXPECT(cache.release_all() == dev.allocs);
    EXPECT(dev.live.empty());
}

void test_full_table_takes_over_the_oldest_slot_through_a_blocking_free() {
    Device dev;
    Cache cache(FakeBackend{&dev});
    bool fresh = false;
    for (int i = 0; i < (int)toa::kPlanSlotsTotal; ++i) {
        Cache::Slot *s = cache.acquire(0, S(i), key_of(1), 1000, &fresh);
        EXPECT(s != nullptr && fresh);
        serve(cache, dev, s, fresh, S(i), key_of(1));
    }
    EXPECT(cache.slots() == toa::kPlanSlotsTotal);
    // stream 0 is still running its launch when a new stream needs a slot
    Cache::Slot *s = cache.acquire(0, S(5000), key_of(1), 1000, &fresh);
    EXPECT(s != nullptr && fresh);           // never "no plan for good"
    EXPECT(s->stream == S(5000));
    EXPECT(dev.blocking_frees == 1);         // stream 0's block went through the blocking free
    serve(cache, dev, s, fresh, S(5000), key_of(1));  // checks: no foreign reader of this memory
    EXPECT(cache.slots() == toa::kPlanSlotsTotal);
    // stream 0 lost its plan and gets a new one by taking over the next oldest (stream 1)
    s = cache.acquire(0, S(0), key_of(1), 1000, &fresh);
    EXPECT(s != nullptr && fresh && s->stream == S(0) && dev.blocking_frees == 2);
}

void test_remembered_calls() {
    Device dev;
    Cache cache(FakeBackend{&dev});
    bool fresh = false;
    Cache::Slot *s = cache.acquire(0, S(0), key_of(1), 1000, &fresh);
    const Bytes call = key_of(42, 64);
    // nothing is remembered for a slot whose contents were never committed
    cache.remember(s, Bytes(call), Memo{1});
    EXPECT(cache.find_call(0, S(0), call) == nullptr);
    serve(cache, dev, s, fresh, S(0), key_of(1));
    cache.remember(s, Bytes(call), Memo{7});
    Cache::Slot *again = cache.find_call(0, S(0), call);
    EXPECT(again == s && again->memo.tag == 7);
    EXPECT(cache.find_call(0, S(1), call) == nullptr);   // another stream: no
    EXPECT(cache.find_call(1, S(0), call) == nullptr);   // another device: no
    EXPECT(cache.find_call(0, S(0), key_of(43, 64)) == nullptr);
    // eviction forgets the call
    for (int k = 2; k < 2 + (int)toa::kPlanSlotsPerStream; ++k) {
        Cache::Slot *t = cache.acquire(0, S(0), key_of(k), 1000, &fresh);
        serve(cache, dev, t, fresh, S(0), key_of(k));
    }
    EXPECT(cache.find_call(0, S(0), call) == nullptr);
    // a failed write leaves neither key nor call behind
    s = cache.acquire(0, S(0), key_of(200), 1000, &fresh);
    cache.invalidate(s);
    cache.acquire(0, S(0), key_of(200), 1000, &fresh);
    EXPECT(fresh);
}

void test_allocation_failure() {
    Device dev;
    FakeBackend backend{&dev};
    backend.fail_alloc = true;
    Cache cache(backend);
    bool fresh = true;
    EXPECT(cache.acquire(0, S(0), key_of(1), 1000, &fresh) == nullptr && !fresh);
    cache.backend().fail_alloc = false;
    Cache::Slot *s = cache.acquire(0, S(0), key_of(1), 1000, &fresh);
    EXPECT(s != nullptr && fresh && cache.slots() == 1);  // the empty slot was taken, not leaked
}

// Several host threads on ONE stream, each bringing lists of its own, more lists than slots:
// between a thread's fill and its launch nobody else may rewrite (or take) the slot.  The
// library holds the cache's mutex over lookup, fill and launch; so does this test.
void test_threads_share_a_stream() {
    Device dev;
    Cache cache(FakeBackend{&dev});
    std::atomic<int> torn{0};
    std::map<void *, int> being_filled;  // block -> thread that is between fill and launch
    auto worker = [&](int id) {
        for (int round = 0; round < 2000; ++round) {
            const Bytes key = key_of(16 * id + round % 7, 8 + (round % 3) * 4096);  // 28 lists
            std::lock_guard<std::mutex> lock(cache.mutex());
            bool fresh = false;
            Cache::Slot *s = cache.acquire(0, S(0), key, key.size() * 8, &fresh);
            if (s == nullptr) continue;
            if (being_filled.count(s->mem)) ++torn;  // somebody else is mid-way on this block
            being_filled[s->mem] = id;
            serve(cache, dev, s, fresh, S(0), key);
            if (s->key != key) ++torn;  // the launch would read another list's records
            being_filled.erase(s->mem);
            if (round % 50 == 0) drain(dev, S(0));
        }
    };
    std::vector<std::thread> threads;
    for (int id = 0; id < 4; ++id) threads.emplace_back(worker, id);
    for (auto &t : threads) t.join();
    EXPECT(torn.load() == 0);
    EXPECT(dev.blocking_frees == 0);
    EXPECT(cache.slots() == toa::kPlanSlotsPerStream);
}

}  // namespace

int main() {
    test_hit_and_lru();
    test_grow_parks_memory_until_its_readers_are_done();
    test_full_table_takes_over_the_oldest_slot_through_a_blocking_free();
    test_remembered_calls();
    test_allocation_failure();
    test_threads_share_a_stream();
    std::printf("ok\n");
    return 0;
}
