// Cache of device-resident plans (per-tensor record tables of long lists), host side only.
//
// The slot state machine is kept apart from the HIP calls it leads to (allocation, events,
// blocking frees come through a Backend) so that it can be driven by a CPU test with a fake
// backend.  No HIP header is included here.
//
// Threading contract.  One mutex guards the whole cache, and the CALLER holds it from the
// lookup until the launch that reads the slot's memory has been enqueued:
//
//     std::lock_guard<std::mutex> lock(cache.mutex());
//     slot = cache.acquire(...);            // may hand back a slot whose contents must be written
//     <enqueue the fill kernels on `stream`>; cache.commit(slot, key) or cache.invalidate(slot)
//     <enqueue the launch that reads slot->mem on `stream`>
//     cache.remember(slot, ...)
//
// A slot's memory is written and read only by work enqueued on the slot's own stream, so stream
// order keeps a rewrite behind every launch that still reads the old contents; holding the mutex
// over lookup, rewrite and launch makes those three one step with respect to other host threads
// (a second thread on the same stream can neither take the slot over between this thread's fill
// and its launch, nor enqueue its own rewrite there).  Memory that a slot outgrows is never
// freed while work may read it: it is parked with an event recorded on its stream and handed out
// again once that event has completed.  Only two things free device memory: release_all(), and
// taking over the slot of ANOTHER stream when the table is full -- both through the backend's
// blocking free, which waits for the device to drain.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <utility>
#include <vector>

namespace toa {

constexpr size_t kPlanSlotsPerStream = 16;  // cached plans a stream may hold
constexpr size_t kPlanSlotsTotal = 128;     // and the process as a whole

// Backend:
//   void *alloc(size_t bytes)                 device memory on the current device, nullptr on failure
//   void free_blocking(int device, void *p)   frees after every stream of `device` has drained
//   bool record(void *stream, Event *out)     an event behind everything enqueued on `stream` so far
//   bool done(const Event &)                  has it completed?  (never blocks)
//   void drop(Event &)                        destroys it
// Memo: what the caller remembers with a slot about the last call it served.
template <class Backend, class Memo>
class PlanCache {
  public:
    using Event = typename Backend::Event;
    using Bytes = std::vector<unsigned char>;

    struct Slot {
        int device = -1;
        void *stream = nullptr;
        void *mem = nullptr;
        size_t capacity = 0;
        Bytes key;   // exact bytes of the records the memory holds; empty: contents unknown
        Bytes call;  // the caller's arguments of the last call served; empty: nothing remembered
        Memo memo{};
        uint64_t stamp = 0;
    };

    explicit PlanCache(Backend backend = Backend()) : backend_(std::move(backend)) {
        slots_.reserve(kPlanSlotsTotal);  // slot addresses stay valid while the mutex is held
    }

    std::mutex &mutex() { return mutex_; }
    Backend &backend() { return backend_; }

    // ---- everything below: the caller holds mutex() ----

    // The slot whose remembered call equals `call`, or nullptr.
    Slot *find_call(int device, void *stream, const Bytes &call) {
        for (Slot &slot : slots_) {
            if (slot.device != device || slot.stream != stream || slot.call.empty() ||
                slot.call != call)
                continue;
            slot.stamp = ++stamp_;
            return &slot;
        }
        return nullptr;
    }

    // The slot that holds (or is to hold) the plan `key` of (device, stream), with memory of at
    // least `need` bytes; nullptr when none can be had.  *fresh says whether the caller must write
    // the contents (on `stream`, before anything reads them) and then commit() or invalidate().
    Slot *acquire(int device, void *stream, const Bytes &key, size_t need, bool *fresh) {
        *fresh = false;
        Slot *oldest_mine = nullptr, *oldest_any = nullptr;
        size_t mine = 0;
        for (Slot &slot : slots_) {
            if (oldest_any == nullptr || slot.stamp < oldest_any->stamp) oldest_any = &slot;
            if (slot.device != device || slot.stream != stream) continue;
            ++mine;
            if (!slot.key.empty() && slot.key == key) {
                slot.stamp = ++stamp_;
                return &slot;
            }
            if (oldest_mine == nullptr || slot.stamp < oldest_mine->stamp) oldest_mine = &slot;
        }
        Slot *use = nullptr;
        bool created = false;
        if (mine >= kPlanSlotsPerStream) {
            use = oldest_mine;  // same stream: its order keeps the rewrite behind the old readers
        } else if (slots_.size() < kPlanSlotsTotal) {
            slots_.emplace_back();
            use = &slots_.back();
            created = true;
        } else {
            // The table is full of other streams' plans (streams since destroyed included): take
            // over the one used longest ago.  Work of its stream may still read its memory, and
            // no event of that stream can be had any more, so the memory goes through the
            // blocking free.
            use = oldest_any;
            if (use->device != device || use->stream != stream) {
                if (use->mem != nullptr) backend_.free_blocking(use->device, use->mem);
                use->mem = nullptr;
                use->capacity = 0;
            }
        }
        use->key.clear();
        use->call.clear();
        if (use->mem != nullptr && use->capacity < need) {
            // outgrown (the slot is this stream's own): launches in flight may still read it
            park(use->device, use->stream, use->mem, use->capacity);
            use->mem = nullptr;
            use->capacity = 0;
        }
        use->device = device;
        use->stream = stream;
        if (use->mem == nullptr) {
            const size_t capacity = need + need / 4;
            use->mem = unpark(device, capacity, &use->capacity);
            if (use->mem == nullptr) {
                use->mem = backend_.alloc(capacity);
                use->capacity = use->mem != nullptr ? capacity : 0;
            }
            if (use->mem == nullptr) {
                if (created)
                    slots_.pop_back();
                else
                    use->stamp = 0;  // an empty slot: the first to be taken over
                return nullptr;
            }
        }
        use->stamp = ++stamp_;
        *fresh = true;
        return use;
    }

    void commit(Slot *slot, Bytes &&key) { slot->key = std::move(key); }
    void invalidate(Slot *slot) {
        slot->key.clear();
        slot->call.clear();
    }
    void remember(Slot *slot, Bytes &&call, const Memo &memo) {
        if (slot->key.empty()) return;
        slot->call = std::move(call);
        slot->memo = memo;
    }

    // Frees everything (blocking).  Returns the number of blocks freed.
    size_t release_all() {
        size_t freed = 0;
        for (Slot &slot : slots_)
            if (slot.mem != nullptr) {
                backend_.free_blocking(slot.device, slot.mem);
                ++freed;
            }
        slots_.clear();
        for (Parked &p : parked_) {
            backend_.free_blocking(p.device, p.mem);
            if (p.has_event) backend_.drop(p.event);
            ++freed;
        }
        parked_.clear();
        return freed;
    }

    size_t slots() const { return slots_.size(); }
    size_t parked() const { return parked_.size(); }
    const Slot &slot(size_t i) const { return slots_[i]; }

  private:
    struct Parked {
        int device;
        void *mem;
        size_t capacity;
        bool has_event;
        Event event;
    };

    void park(int device, void *stream, void *mem, size_t capacity) {
        Parked p{device, mem, capacity, false, Event{}};
        p.has_event = backend_.record(stream, &p.event);
        if (!p.has_event) {
            // no event to wait on: nothing can vouch for this block, so it goes the slow way
            backend_.free_blocking(device, mem);
            return;
        }
        parked_.push_back(p);
    }

    // A parked block of `device` with at least `bytes` that nothing reads any more.
    void *unpark(int device, size_t bytes, size_t *capacity) {
        for (size_t i = 0; i < parked_.size(); ++i) {
            Parked &p = parked_[i];
            if (p.device != device || p.capacity < bytes || !backend_.done(p.event)) continue;
            void *mem = p.mem;
            *capacity = p.capacity;
            backend_.drop(p.event);
            parked_[i] = parked_.back();
            parked_.pop_back();
            return mem;
        }
        return nullptr;
    }

    Backend backend_;
    std::mutex mutex_;
    std::vector<Slot> slots_;
    std::vector<Parked> parked_;
    uint64_t stamp_ = 0;
};

}  // namespace toa
