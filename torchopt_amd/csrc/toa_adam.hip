// Host side of libtoa_adam.so: the C ABI declared in include/toa_adam.h.
//
// Each entry point rounds the Python-level scalars the way the reference
// launchers do (/root/reference/src/adam_op/adam_op_impl_cpu.cpp:73-84,
// 191-206, 328-343: powers, differences and reciprocals in double, then one
// cast to the element type), picks a grid and enqueues one kernel on the
// caller's stream.  Nothing here copies or synchronises, and the single-tensor
// entry points allocate nothing; the list entry points keep the record tables
// of long lists ("plans") in device memory that the library allocates once per
// (device, stream, list) and caches (plan_cache.hpp) -- except
// toa_adam_forward_inplace_multi_noalloc, whose plan lives in a file-scope
// device array.
#include "toa_adam.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <vector>

#include "adam_kernels.hpp"
#include "plan_cache.hpp"

// Bytes of the file-scope plan array behind toa_adam_forward_inplace_multi_noalloc: 4096 records
// of 96 bytes and, behind them, the finer tile index of a long list (at most four 4-byte entries
// per record).
constexpr size_t toa_noalloc_scratch_bytes = 4096 * 96 + 4 * 4096 * 4;

namespace {

using namespace toa;

// Launch shape of the streaming kernels (see adam_kernels.hpp).
constexpr int kUnroll = 1;           // one 16-byte access per lane per stream
constexpr bool kNonTemporal = true;  // every array is touched once
constexpr unsigned kMaxGrid = 1u << 25;  // default cap on workgroups per launch
// LDS of a gfx950 compute unit: 160 KiB handed out in granules of 1280 bytes (128 per CU).  A
// single-wave workgroup that reserves g granules therefore limits residency to floor(128 / g)
// workgroups per CU: 32 (no reservation; the wave-slot limit), 25, 21, 18, 16, 14, 12, 11, 10,
// 9, 8 ...  Measured on MI355X with a kernel that counts its concurrently resident workgroups:
// 12 800 bytes -> 12 per CU, 12 801 -> 11; 6 400 -> 25, 6 401 -> 21.
constexpr int kLdsGranule = 1280;
constexpr int kLdsGranulesPerCU = 128;
constexpr int kMaxWavesPerCU = 32;
// One workgroup per CU would need 83 200 bytes of dynamic LDS, more than the 64 KiB a launch may
// reserve without raising the kernel's limit; two per CU (55 040 bytes) is the lowest level served.
constexpr int kMinWavesPerCU = 2;

// Global override of the per-op resident-wave cap: -1 = not yet initialised,
// 0 = use each op's own kWavesPerCU, 2..32 = that many for every op.  Set by
// toa_adam_set_waves_per_cu() or, initially, by the environment variable
// TOA_ADAM_WAVES_PER_CU (read once).
std::atomic<int> g_waves_override{-1};

int waves_override() {
    int w = g_waves_override.load(std::memory_order_relaxed);
    if (w < 0) {
        w = 0;
        if (const char *env = std::getenv("TOA_ADAM_WAVES_PER_CU")) {
            const int v = std::atoi(env);
            if (v >= kMinWavesPerCU && v <= kMaxWavesPerCU) w = v;
        }
        g_waves_override.store(w, std::memory_order_relaxed);
    }
    return w;
}

// Dynamic LDS bytes that hold residency to the largest achievable level not above `waves`
// single-wave workgroups per CU.  The kernels never touch LDS; the reservation only bounds
// residency.
constexpr unsigned lds_for_waves(int waves) {
    if (waves >= kMaxWavesPerCU) return 0;
    if (waves < 1) waves = 1;
    // smallest g with floor(128 / g) <= waves
    return (unsigned)((kLdsGranulesPerCU / (waves + 1) + 1) * kLdsGranule);
}
static_assert(lds_for_waves(12) == 12800 && lds_for_waves(13) == 12800, "12 per CU");
static_assert(lds_for_waves(14) == 11520 && lds_for_waves(16) == 10240, "14 and 16 per CU");
static_assert(lds_for_waves(25) == 6400 && lds_for_waves(24) == 7680, "25 and 21 per CU");
static_assert(lds_for_waves(31) == 6400 && lds_for_waves(32) == 0, "25, then no reservation");
static_assert(lds_for_waves(1) == 65 * 1280, "one per CU: more than half of the LDS");
static_assert(lds_for_waves(kMinWavesPerCU) <= 64 * 1024, "every served level fits a launch");

// The multi-tensor kernel spends three dependent scalar loads finding its tensor before any
// memory traffic starts, so its best level sits one or two steps above the single-tensor one.
// A launch that fits on the chip in one round (256 CUs x 32 wave slots) is latency-bound, not
// bandwidth-bound: capping residency would only add rounds (2^21 float32 elements in place:
// 8.8 us capped, 6.5 us uncapped), so such launches run without a reservation.
constexpr size_t kOneRoundTiles = 256 * kMaxWavesPerCU;

// Residency level of a staged list launch: the op's own figure where it was measured, else the
// single-tensor level.
template <class Op, class = void>
struct StagedListLevel {
    static constexpr int value = Op::kWavesPerCUStaged;
};
template <class Op>
struct StagedListLevel<Op, decltype((void)Op::kWavesPerCUStagedLists)> {
    static constexpr int value = Op::kWavesPerCUStagedLists;
};
template <class Op>
constexpr int staged_list_level() {
    return StagedListLevel<Op>::value;
}

template <class Op>
unsigned lds_reservation(bool multi, size_t num_tiles, bool staged = false) {
    const int o = waves_override();
    if (o) return lds_for_waves(o);
    if (num_tiles <= kOneRoundTiles) return 0;
    if constexpr (IsStaged<Op>::value) {
        if (staged) return lds_for_waves(multi ? staged_list_level<Op>() : Op::kWavesPerCUStaged);
    }
    return lds_for_waves(multi ? Op::kWavesPerCUMulti : Op::kWavesPerCU);
}

// Schedule of the ops that have a staged form (see tile_full_staged): 0 = the measured choice
// (single tensors staged, lists staged when their arrays collide in DRAM), 1 = never staged,
// 2 = staged wherever it is legal.  The staged schedule stores early results before the last
// input is loaded, so it needs the arrays of a tensor to be disjoint; overlapping arrays (the
// reference's availability probe passes one array three times) take the plain schedule.
std::atomic<int> g_schedule{0};

// Load order of the staged program of big single-tensor launches (ops that have several, see
// LoadOrders): -1 = the library's choice, 0 .. 3 = that order wherever the op has it.
std::atomic<int> g_load_order{-1};

// Arrays of one tensor whose addresses differ by (nearly) a multiple of 16 MiB meet in the same
// DRAM banks: measured on MI355X the in-place step falls from 6.6 to 5.5-6.1 TB/s when the
// distance is within 1.5 MiB of such a multiple (GPT-2-medium's 4096 x 1024 float32 weights are
// exactly 16 MiB).  The staged schedule at a low residency level recovers most of it.
template <typename T, int NPTR>
bool arrays_collide(T *const (&ptrs)[NPTR], size_t n) {
    constexpr uintptr_t kPeriod = (uintptr_t)16 << 20, kNear = (uintptr_t)3 << 19;
    if (n * sizeof(T) < ((size_t)4 << 20)) return false;  // small arrays sit in cache
    for (int i = 0; i < NPTR; ++i)
        for (int j = i + 1; j < NPTR; ++j) {
            const uintptr_t a = reinterpret_cast<uintptr_t>(ptrs[i]);
            const uintptr_t b = reinterpret_cast<uintptr_t>(ptrs[j]);
            const uintptr_t d = (a < b ? b - a : a - b) % kPeriod;
            if (d < kNear || kPeriod - d < kNear) return true;
        }
    return false;
}

template <typename T, int NPTR>
bool arrays_disjoint(T *const (&ptrs)[NPTR], size_t n) {
    const size_t bytes = n * sizeof(T);
    for (int i = 0; i < NPTR; ++i)
        for (int j = i + 1; j < NPTR; ++j) {
            const uintptr_t a = reinterpret_cast<uintptr_t>(ptrs[i]);
            const uintptr_t b = reinterpret_cast<uintptr_t>(ptrs[j]);
            if (a < b ? b - a < bytes : a - b < bytes) return false;
        }
    return true;
}

// Where first moments should begin, as an address modulo kStatePeriod; second moments begin at
// a multiple of it (see toa_adam_state_shift).
constexpr uintptr_t kStatePeriod = 16 << 10, kStatePhase = 8 << 10;

// Workgroups per launch are capped; a tensor with more tiles than the cap is covered by the
// kernels' stride loop.  The cap is adjustable so that path can be exercised on small inputs.
std::atomic<unsigned> g_max_grid{kMaxGrid};

unsigned grid_for(size_t num_tiles) {
    const unsigned cap = g_max_grid.load(std::memory_order_relaxed);
    return (unsigned)(num_tiles < cap ? num_tiles : cap);
}

struct HostScalars {
    double c1, c2, p1, q2;
};

// adam_op_impl_cpu.cpp:73-74 (c1, c2), :328-329 (p1, q2); std::pow(double, size_t)
// promotes the exponent to double.
HostScalars host_scalars(double b1, double b2, double eps_root, uint64_t count) {
    const double pb1 = std::pow(b1, (double)count);
    const double pb2 = std::pow(b2, (double)count);
    return {1 / (1 - pb1), 1 / (1 - pb2), 1 - pb1, 1 / (1 - pb2 + eps_root)};
}

// The device-side step reference of the *_devcount entry points, checked.
template <typename T>
int make_step_ref(const void *bias_rows, uint64_t first_count, size_t rows, const int64_t *count,
                  StepRef<T> *out) {
    if (bias_rows == nullptr || count == nullptr) return TOA_ENULL;
    if (rows == 0 || rows > ((size_t)1 << 40) || first_count > (uint64_t)INT64_MAX) return TOA_ESIZE;
    *out = StepRef<T>{static_cast<const T *>(bias_rows), count, (int64_t)first_count,
                      (int64_t)rows - 1};
    return 0;
}

// One address per op type: tells the remembered calls of different ops apart.
template <class Op>
struct OpTag {
    static const char tag;
};
template <class Op>
const char OpTag<Op>::tag = 0;

// ---------------------------------------------------------------------------
// Which load order a big single-tensor staged launch runs, chosen per call site by measurement.
//
// How three read and three write streams fall on the memory channels depends on where the three
// arrays lie, and with it which of the four load orders of the staged program streams fastest:
// on most placements the first (g, mu, nu) does, on some another gains 1-2 %.  The results are
// the same bits in every order, so the library can try them on the caller's own launches: the
// first kTuneRounds x 5 launches of a call site (one op on one set of arrays of one length) go
// round the four orders and the plain schedule (all loads, then all stores at its own residency
// level: on a few placements -- both moments 4 KiB off the gradient's phase is one -- it beats
// every staged order by 1-2 %), timed with events on the caller's stream; rounds alternate their
// direction and the first two do not count, so a drift in the machine's rate (clocks settling
// under a new load) cancels instead of favouring whatever ran last.  Once every sample has come
// back -- events are polled, never waited for -- the variant with the lowest mean time is kept for
// the call site if it beats the default order by more than kTuneMargin, the default otherwise.
// Nothing is tuned under stream capture, with an order or residency level forced, or with
// tuning switched off; up to kTuneSites call sites are remembered, least recently used first out.
// ---------------------------------------------------------------------------
constexpr int kTuneOrders = 4;    // load orders of the staged program
constexpr int kTuneVariants = 5;  // ... and the plain schedule (all loads, then all stores)
constexpr int kTunePlain = 4;
constexpr int kTuneRounds = 6, kTuneSkippedRounds = 2;
constexpr double kTuneMargin = 0.004;
constexpr size_t kTuneSites = 64;
constexpr size_t kTuneFromBytes = (size_t)64 << 20;  // per array: launches of 60 us and more

std::atomic<int> g_tuning{-1};  // -1 = not yet initialised, 0 = off, 1 = on

bool tuning_on() {
    int t = g_tuning.load(std::memory_order_relaxed);
    if (t < 0) {
        const char *env = std::getenv("TOA_ADAM_TUNING");
        t = (env != nullptr && env[0] == '0') ? 0 : 1;
        g_tuning.store(t, std::memory_order_relaxed);
    }
    return t != 0;
}

struct TuneSite {
    const void *tag = nullptr;  // the op
    uintptr_t p[3] = {0, 0, 0};
    size_t n = 0;
    int device = 0;
    uint64_t stamp = 0;
    int decided = -1;  // the variant kept (0-3 an order, 4 plain), or -1 while being explored
    int launches = 0;  // exploring launches issued so far
    double sum[kTuneVariants] = {0, 0, 0, 0, 0};
    int count[kTuneVariants] = {0, 0, 0, 0, 0};
    struct Sample {
        int order;
        bool counted;
        hipEvent_t begin, end;
    };
    std::vector<Sample> pending;
};
std::mutex g_tune_mutex;
std::vector<TuneSite> g_tune_sites;
uint64_t g_tune_stamp = 0;

void tune_drop_events(TuneSite &site) {
    for (TuneSite::Sample &s : site.pending) {
        (void)hipEventDestroy(s.begin);
        (void)hipEventDestroy(s.end);
    }
    site.pending.clear();
}

// Collects the samples that have come back; decides once all have.  g_tune_mutex held.
void tune_collect(TuneSite &site) {
    size_t kept = 0;
    for (size_t i = 0; i < site.pending.size(); ++i) {
        TuneSite::Sample &s = site.pending[i];
        const hipError_t ready = hipEventQuery(s.end);
        if (ready == hipErrorNotReady) {
            (void)hipGetLastError();
            site.pending[kept++] = s;
            continue;
        }
        float ms = 0.0f;
        if (ready == hipSuccess && hipEventElapsedTime(&ms, s.begin, s.end) == hipSuccess) {
            if (s.counted && ms > 0.0f) {
                site.sum[s.order] += ms;
                ++site.count[s.order];
            }
        } else {
            (void)hipGetLastError();
        }
        (void)hipEventDestroy(s.begin);
        (void)hipEventDestroy(s.end);
    }
    site.pending.resize(kept);
    if (site.launches < kTuneRounds * kTuneVariants || !site.pending.empty()) return;
    int best = 0;
    bool complete = true;
    double mean[kTuneVariants];
    for (int o = 0; o < kTuneVariants; ++o) {
        complete = complete && site.count[o] == kTuneRounds - kTuneSkippedRounds;
        mean[o] = site.count[o] ? site.sum[o] / site.count[o] : 0.0;
    }
    if (complete)
        for (int o = 1; o < kTuneVariants; ++o)
            if (mean[o] < mean[best]) best = o;
    site.decided = (complete && mean[best] < mean[0] * (1.0 - kTuneMargin)) ? best : 0;
}

TuneSite *tune_find(const void *tag, const uintptr_t (&p)[3], size_t n, int device, bool create) {
    TuneSite *oldest = nullptr;
    for (TuneSite &site : g_tune_sites) {
        if (site.tag == tag && site.n == n && site.device == device && site.p[0] == p[0] &&
            site.p[1] == p[1] && site.p[2] == p[2]) {
            site.stamp = ++g_tune_stamp;
            return &site;
        }
        if (oldest == nullptr || site.stamp < oldest->stamp) oldest = &site;
    }
    if (!create) return nullptr;
    TuneSite *site = oldest;
    if (g_tune_sites.size() < kTuneSites) {
        g_tune_sites.emplace_back();
        site = &g_tune_sites.back();
    } else {
        tune_drop_events(*site);
        *site = TuneSite();
    }
    site->tag = tag;
    for (int i = 0; i < 3; ++i) site->p[i] = p[i];
    site->n = n;
    site->device = device;
    site->stamp = ++g_tune_stamp;
    return site;
}

// The staged whole-tile kernel in one of the op's load orders.
template <typename T, class Op>
void launch_full_staged(int order, const Op &op, const TensorPtrs<T, Op> &tp, size_t whole,
                        unsigned lds, void *stream) {
    auto go = [&](auto ORDER) {
        hipLaunchKernelGGL(
            (full_tiles_kernel<T, Op, kUnroll, kNonTemporal, true, decltype(ORDER)::value>),
            dim3((unsigned)whole), dim3(kBlock), lds, (hipStream_t)stream, op, tp);
    };
    if constexpr (LoadOrders<Op>::value == 4) {
        switch (order) {
            case 1: return go(std::integral_constant<int, 1>{});
            case 2: return go(std::integral_constant<int, 2>{});
            case 3: return go(std::integral_constant<int, 3>{});
            default: break;
        }
    }
    go(std::integral_constant<int, 0>{});
}

// A big staged launch of an op with several load orders, at the order its call site has settled
// on, or -- while the site is being explored -- at the next order to try, timed.  False when the
// launch is not the tuner's to make (the stream is capturing, no device).
template <typename T, class Op>
bool launch_tuned(const Op &op, const TensorPtrs<T, Op> &tp, size_t whole, unsigned lds,
                  void *stream) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    int device = 0;
    if (hipStreamIsCapturing((hipStream_t)stream, &capturing) != hipSuccess ||
        capturing != hipStreamCaptureStatusNone || hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    const uintptr_t p[3] = {reinterpret_cast<uintptr_t>(tp.p[0]),
                            reinterpret_cast<uintptr_t>(tp.p[1]),
                            reinterpret_cast<uintptr_t>(tp.p[2])};
    std::unique_lock<std::mutex> lock(g_tune_mutex);
    TuneSite *site = tune_find(&OpTag<Op>::tag, p, whole, device, true);
    if (site->decided < 0) tune_collect(*site);
    // one variant of the five: a load order of the staged program, or the plain schedule
    auto launch_variant = [&](int variant) {
        if (variant == kTunePlain)
            hipLaunchKernelGGL((full_tiles_kernel<T, Op, kUnroll, kNonTemporal>),
                               dim3((unsigned)whole), dim3(kBlock), lds_reservation<Op>(false, whole),
                               (hipStream_t)stream, op, tp);
        else
            launch_full_staged<T, Op>(variant, op, tp, whole, lds, stream);
    };
    if (site->decided >= 0 || site->launches >= kTuneRounds * kTuneVariants) {
        // settled, or every exploring launch is out and its samples are still on their way
        const int variant = site->decided >= 0 ? site->decided : 0;
        lock.unlock();
        launch_variant(variant);
        return true;
    }
    const int round = site->launches / kTuneVariants, at = site->launches % kTuneVariants;
    TuneSite::Sample sample;
    sample.order = round % 2 == 0 ? at : kTuneVariants - 1 - at;
    sample.counted = round >= kTuneSkippedRounds;
    ++site->launches;
    const bool timed = hipEventCreate(&sample.begin) == hipSuccess &&
                       (hipEventCreate(&sample.end) == hipSuccess ||
                        (hipEventDestroy(sample.begin), false));
    if (!timed) (void)hipGetLastError();
    // record, launch, record: one step under the mutex, so no other launch of the library lands
    // between the two events on this stream.  An event that fails costs the sample, never the
    // launch: its error is cleared, so that the caller reports the launch's own status alone.
    bool recorded = timed && hipEventRecord(sample.begin, (hipStream_t)stream) == hipSuccess;
    if (timed && !recorded) (void)hipGetLastError();
    launch_variant(sample.order);
    const hipError_t launch_rc = hipPeekAtLastError();
    if (recorded && hipEventRecord(sample.end, (hipStream_t)stream) != hipSuccess) {
        recorded = false;
        if (launch_rc == hipSuccess) (void)hipGetLastError();
    }
    if (recorded && launch_rc == hipSuccess) {
        site->pending.push_back(sample);
    } else if (timed) {
        (void)hipEventDestroy(sample.begin);
        (void)hipEventDestroy(sample.end);
    }
    return true;
}

template <typename T, class Op>
int launch_single(const Op &op, T *const (&ptrs)[Op::NPTR], size_t n, void *stream) {
    if (n == 0) return 0;
    TensorPtrs<T, Op> tp;
    for (int i = 0; i < Op::NPTR; ++i) {
        if (ptrs[i] == nullptr) return TOA_ENULL;
        tp.p[i] = ptrs[i];
    }
    constexpr size_t tile = Tile<T, kUnroll>::ELEMS;
    // Bandwidth-bound launches with aligned operands: the whole tiles go to the branch-free
    // kernel, one workgroup each, and a ragged last tile to the general kernel.  Launches of one
    // round of workgroups (latency-bound: a second launch would cost more than the branches),
    // tensors beyond the grid cap and unaligned operands take the general kernel alone.
    uintptr_t bits = 0;
    for (int i = 0; i < Op::NPTR; ++i) bits |= reinterpret_cast<uintptr_t>(ptrs[i]);
    const size_t whole = n / tile;
    if ((bits & 15u) == 0 && whole > kOneRoundTiles &&
        whole <= g_max_grid.load(std::memory_order_relaxed)) {
        bool staged = false;
        if constexpr (IsStaged<Op>::value)
            staged = g_schedule.load(std::memory_order_relaxed) != 1 && arrays_disjoint(ptrs, n);
        if (staged) {
            if constexpr (IsStaged<Op>::value) {
                const unsigned lds = lds_reservation<Op>(false, whole, true);
                int order = g_load_order.load(std::memory_order_relaxed);
                bool launched = false;
                if constexpr (LoadOrders<Op>::value == kTuneOrders && Op::NPTR == 3) {
                    if (order < 0 && tuning_on() && waves_override() == 0 &&
                        g_schedule.load(std::memory_order_relaxed) == 0 &&
                        whole * tile * sizeof(T) >= kTuneFromBytes)
                        launched = launch_tuned<T, Op>(op, tp, whole, lds, stream);
                }
                if (!launched) {
                    if (order < 0 || order >= LoadOrders<Op>::value) order = 0;
                    launch_full_staged<T, Op>(order, op, tp, whole, lds, stream);
                }
            }
        } else {
            hipLaunchKernelGGL((full_tiles_kernel<T, Op, kUnroll, kNonTemporal>),
                               dim3((unsigned)whole), dim3(kBlock),
                               lds_reservation<Op>(false, whole), (hipStream_t)stream, op, tp);
        }
        if (const int rc = (int)hipGetLastError()) return rc;
        const size_t done = whole * tile;
        if (done == n) return 0;
        for (int i = 0; i < Op::NPTR; ++i) tp.p[i] += done;
        n -= done;
    }
    const size_t num_tiles = (n + tile - 1) / tile;
    hipLaunchKernelGGL((stream_kernel<T, Op, kUnroll, kNonTemporal>), dim3(grid_for(num_tiles)),
                       dim3(kBlock), lds_reservation<Op>(false, num_tiles), (hipStream_t)stream,
                       op, tp, n, num_tiles);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Plans: device-resident tables for lists longer than one kernel-argument table.
// ---------------------------------------------------------------------------

// 0 = plans for lists that need more than one kernel-argument table (the default), 1 = never
// (several launches instead), 2 = for every list (so that small inputs can exercise the path).
std::atomic<int> g_plan_mode{0};
constexpr uint64_t kPlanFromTiles = 1u << 18;  // 256 MiB of 1 KiB tiles per array

// A plan of more than kPlanFineFrom records carries a finer index behind its records: one entry
// per 2^shift tiles, the smallest shift that leaves at most four entries per record.
constexpr size_t kPlanFineFrom = 2 * kPlanCells;

uint32_t plan_fine_entries(size_t num, uint64_t total_tiles, uint32_t *shift) {
    *shift = 0;
    if (num <= kPlanFineFrom) return 0;
    while (((total_tiles + ((uint64_t)1 << *shift) - 1) >> *shift) > 4 * (uint64_t)num) ++*shift;
    return (uint32_t)((total_tiles + ((uint64_t)1 << *shift) - 1) >> *shift);
}

size_t plan_record_bytes(size_t num) { return (num * sizeof(PlanRec) + 255) / 256 * 256; }
// records, then the finer index (if any)
size_t plan_bytes(size_t num, uint32_t fine_entries) {
    return plan_record_bytes(num) + (size_t)fine_entries * sizeof(uint32_t);
}

// Writes the records for `seeds` into `mem` (device memory of at least plan_record_bytes(seeds.size()))
// on `stream`: fill kernels carrying the records in their arguments.
template <int NPTR>
int plan_write(void *mem, const std::vector<PlanSeed<NPTR>> &seeds, hipStream_t stream) {
    using Chunk = PlanSeedChunk<NPTR>;
    PlanRec *recs = static_cast<PlanRec *>(mem);
    const uint32_t num = (uint32_t)seeds.size();
    Chunk chunk;
    for (uint32_t at = 0; at < num; at += Chunk::MAX) {
        const uint32_t count = num - at < (uint32_t)Chunk::MAX ? num - at : Chunk::MAX;
        std::memcpy(chunk.seed, seeds.data() + at, count * sizeof(PlanSeed<NPTR>));
        hipLaunchKernelGGL((plan_fill_kernel<NPTR>), dim3(1), dim3(128), 0, stream, recs, at,
                           count, chunk);
        if (const int rc = (int)hipGetLastError()) return rc;
    }
    return 0;
}

// The records and, for a plan of more than kPlanFineFrom records, the finer index behind them.
template <int NPTR>
int plan_write_all(void *mem, const std::vector<PlanSeed<NPTR>> &seeds, uint32_t fine_entries,
                   uint32_t fine_shift, hipStream_t stream) {
    if (const int rc = plan_write<NPTR>(mem, seeds, stream)) return rc;
    if (fine_entries == 0) return 0;
    hipLaunchKernelGGL(plan_index_kernel, dim3((fine_entries + 255) / 256), dim3(256), 0, stream,
                       static_cast<const PlanRec *>(mem), (uint32_t)seeds.size(),
                       reinterpret_cast<uint32_t *>(static_cast<char *>(mem) +
                                                    plan_record_bytes(seeds.size())),
                       fine_entries, fine_shift);
    return (int)hipGetLastError();
}

// The launch's view of a plan: the coarse index from tile cells to records, and the finer one in
// device memory where the plan has it (lists of more than kPlanFineFrom records).
template <int NPTR>
PlanView plan_view(void *mem, const std::vector<PlanSeed<NPTR>> &seeds, uint32_t total) {
    PlanView v;
    v.recs = static_cast<const PlanRec *>(mem);
    v.total = total;
    v.num = (uint32_t)seeds.size();
    v.fine = nullptr;
    v.fine_shift = 0;
    if (plan_fine_entries(seeds.size(), total, &v.fine_shift) != 0)
        v.fine = reinterpret_cast<const uint32_t *>(static_cast<const char *>(mem) +
                                                   plan_record_bytes(seeds.size()));
    v.shift = 0;
    while ((((uint64_t)total + (1u << v.shift) - 1) >> v.shift) > (uint64_t)kPlanCells) ++v.shift;
    uint32_t k = 0;
    for (uint32_t c = 0; c < (uint32_t)kPlanCells; ++c) {
        const uint64_t tile = (uint64_t)c << v.shift;
        while (k + 1 < v.num && seeds[k].next_first <= tile) ++k;
        v.cell[c] = k;
    }
    return v;
}

// Cached plans (plan_cache.hpp holds the slot state machine and its threading contract): keyed by
// (device, stream, exact bytes of the records).  A slot also remembers the last call it served,
// whole -- the caller's arguments as bytes and the launch they led to.  A training loop calls with
// the same lists step after step; when the arguments are byte for byte those of the last time,
// every per-tensor decision is known already and the call is one comparison and one launch
// (150 ns per tensor otherwise).
struct PlanMemo {
    PlanView view;
    bool staged = false;
};

struct HipPlanBackend {
    using Event = hipEvent_t;
    void *alloc(size_t bytes) {
        void *p = nullptr;
        if (hipMalloc(&p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        return p;
    }
    void free_blocking(int device, void *p) {  // hipFree waits for the device to drain
        int current = 0;
        (void)hipGetDevice(&current);
        if (current != device) (void)hipSetDevice(device);
        if (hipFree(p) != hipSuccess) (void)hipGetLastError();
        if (current != device) (void)hipSetDevice(current);
    }
    bool record(void *stream, Event *out) {
        if (hipEventCreateWithFlags(out, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        if (hipEventRecord(*out, (hipStream_t)stream) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipEventDestroy(*out);
            return false;
        }
        return true;
    }
    bool done(const Event &e) {
        if (hipEventQuery(e) == hipSuccess) return true;
        (void)hipGetLastError();  // "not ready" is an answer, not an error to leave behind
        return false;
    }
    void drop(Event &e) { (void)hipEventDestroy(e); }
};

using Plans = PlanCache<HipPlanBackend, PlanMemo>;
Plans g_plans;

// Called with g_plans.mutex() held.  Returns the slot whose device memory holds the plan for
// `seeds`, written on `stream` if it was not already there; nullptr when no plan can be had (the
// caller then launches table by table).  The caller enqueues its launch before it lets go of the
// mutex.
template <int NPTR>
Plans::Slot *plan_cached(const std::vector<PlanSeed<NPTR>> &seeds, size_t tile, int device,
                         hipStream_t stream, int *rc) {
    *rc = 0;
    Plans::Bytes key(16 + seeds.size() * sizeof(PlanSeed<NPTR>));
    const uint64_t head[2] = {(uint64_t)NPTR, (uint64_t)tile};
    std::memcpy(key.data(), head, 16);
    std::memcpy(key.data() + 16, seeds.data(), seeds.size() * sizeof(PlanSeed<NPTR>));

    const uint64_t total_tiles = seeds.empty() ? 0 : seeds.back().next_first;
    uint32_t fine_shift = 0;
    const uint32_t fine_entries = plan_fine_entries(seeds.size(), total_tiles, &fine_shift);
    bool fresh = false;
    Plans::Slot *slot = g_plans.acquire(device, (void *)stream, key,
                                        plan_bytes(seeds.size(), fine_entries), &fresh);
    if (slot == nullptr || !fresh) return slot;
    *rc = plan_write_all<NPTR>(slot->mem, seeds, fine_entries, fine_shift, stream);
    if (*rc) {
        g_plans.invalidate(slot);
        return nullptr;
    }
    g_plans.commit(slot, std::move(key));
    return slot;
}

// Memory for the plan of one call, brought by the caller instead of taken from the cache (the
// entry point that must not allocate).  The plan is rewritten on every call.
struct PlanArena {
    void *mem = nullptr;
    size_t bytes = 0;
};

// Launch one op over a list of tensors.  `make_op(count)` builds the op's scalars for one step
// number; tensors are batched per distinct count.  A batch that fits one kernel-argument table
// is one launch with the table in its arguments; a longer one is one launch over a
// device-resident plan (cached per stream and list), or -- where no plan can be had: under
// stream capture, or with plans switched off -- one launch per table.
template <typename T, class Op, class MakeOp>
int launch_multi(MakeOp make_op, size_t num_tensors,
                 const void *const *const (&lists)[Op::NPTR],
                 const size_t *n, const uint64_t *counts, uint64_t count_all, void *stream,
                 const PlanArena *arena = nullptr) {
    using Table = MultiTable<T, Op>;
    // HIP allows 4 KiB of kernel arguments, 256 bytes of them implicit
    static_assert(sizeof(Op) + sizeof(Table) + 256 <= 4096, "table launch fits its arguments");
    static_assert(sizeof(Op) + sizeof(PlanView) + 256 <= 4096, "plan launch fits its arguments");
    constexpr size_t tile = Tile<T, kUnroll>::ELEMS;
    if (num_tensors == 0) return 0;
    if (n == nullptr) return TOA_ENULL;
    for (int i = 0; i < Op::NPTR; ++i)
        if (lists[i] == nullptr) return TOA_ENULL;

    // A call whose arguments are byte for byte those a cached plan last served: one launch.
    // (One step count for the whole list, the caller not capturing, plans not switched off;
    // everything else -- validation, schedule, plan -- was settled when the call was first seen.)
    std::vector<unsigned char> call;
    if (counts == nullptr && arena == nullptr && g_plan_mode.load(std::memory_order_relaxed) != 1) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing((hipStream_t)stream, &capturing) == hipSuccess &&
            capturing == hipStreamCaptureStatusNone) {
            const uint64_t head[4] = {reinterpret_cast<uintptr_t>(&OpTag<Op>::tag),
                                      (uint64_t)g_schedule.load(std::memory_order_relaxed),
                                      (uint64_t)g_plan_mode.load(std::memory_order_relaxed),
                                      (uint64_t)num_tensors};
            static_assert(sizeof(size_t) == sizeof(void *), "sizes and pointers copy alike");
            const size_t row = num_tensors * sizeof(void *);
            call.resize(sizeof(head) + (Op::NPTR + 1) * row);
            unsigned char *at = call.data();
            std::memcpy(at, head, sizeof(head));
            at += sizeof(head);
            // pointers first: two lists of one model differ there, not in their sizes, so a
            // comparison with another list's remembered call ends at its first bytes
            for (int i = 0; i < Op::NPTR; ++i, at += row) std::memcpy(at, lists[i], row);
            std::memcpy(at, n, row);
            int device = 0;
            if (hipGetDevice(&device) == hipSuccess) {
                // lookup and launch are one step under the cache's mutex (plan_cache.hpp)
                std::lock_guard<std::mutex> lock(g_plans.mutex());
                if (Plans::Slot *slot = g_plans.find_call(device, stream, call)) {
                    const PlanView &view = slot->memo.view;
                    const bool staged_before = slot->memo.staged;
                    const Op op = make_op(count_all);
                    const unsigned lds =
                        lds_reservation<Op>(staged_before, view.total, staged_before);
                    if (staged_before) {
                        if constexpr (IsStaged<Op>::value)
                            hipLaunchKernelGGL(
                                (plan_stream_kernel<T, Op, kUnroll, kNonTemporal, true>),
                                dim3(grid_for(view.total)), dim3(kBlock), lds, (hipStream_t)stream,
                                op, view);
                    } else {
                        hipLaunchKernelGGL((plan_stream_kernel<T, Op, kUnroll, kNonTemporal>),
                                           dim3(grid_for(view.total)), dim3(kBlock), lds,
                                           (hipStream_t)stream, op, view);
                    }
                    return (int)hipGetLastError();
                }
            }
        } else {
            (void)hipGetLastError();
        }
    }

    // validate everything before the first launch
    for (size_t k = 0; k < num_tensors; ++k) {
        if (n[k] == 0) continue;
        for (int i = 0; i < Op::NPTR; ++i)
            if (lists[i][k] == nullptr) return TOA_ENULL;
        if ((n[k] + tile - 1) / tile > 0x7fffffffu) return TOA_ESIZE;
    }

    // A list takes the staged schedule when the op gains from it on any list (kStagedLists), or
    // when a quarter or more of its elements belong to tensors whose arrays collide in DRAM (it
    // then runs 12 % faster) -- and every tensor's arrays are disjoint, which the schedule needs.
    bool staged = false;
    if constexpr (IsStaged<Op>::value) {
        const int schedule = g_schedule.load(std::memory_order_relaxed);
        if (schedule != 1) {
            size_t total = 0, colliding = 0;
            bool disjoint = true;
            for (size_t k = 0; disjoint && k < num_tensors; ++k) {
                if (n[k] == 0) continue;
                T *p[Op::NPTR];
                for (int i = 0; i < Op::NPTR; ++i)
                    p[i] = static_cast<T *>(const_cast<void *>(lists[i][k]));
                T *const(&cp)[Op::NPTR] = p;
                disjoint = arrays_disjoint(cp, n[k]);
                total += n[k];
                if (arrays_collide(cp, n[k])) colliding += n[k];
            }
            staged = disjoint && (schedule == 2 || Op::kStagedLists || colliding * 4 >= total);
        }
    }

    std::vector<uint64_t> distinct;
    if (counts == nullptr) {
        distinct.push_back(count_all);
    } else {
        for (size_t k = 0; k < num_tensors; ++k) {
            if (n[k] == 0) continue;
            bool seen = false;
            for (uint64_t c : distinct) seen |= (c == counts[k]);
            if (!seen) distinct.push_back(counts[k]);
        }
    }

    const int plan_mode = g_plan_mode.load(std::memory_order_relaxed);
    std::vector<PlanSeed<Op::NPTR>> seeds;
    Table tab;
    uint32_t num = 0;       // tensors in the table being filled
    uint32_t next_tile = 0; // tiles in the table being filled
    auto reset = [&]() {
        num = 0;
        next_tile = 0;
        for (int g = 0; g < kMaxGroups; ++g) tab.coarse[g] = kNoTile;
        for (int g = 0; g < Table::GROUPS; ++g)
            for (int i = 0; i < kGroup; ++i) tab.group[g].start[i] = kNoTile;
    };
    for (uint64_t c : distinct) {
        const Op op = make_op(c);
        auto member = [&](size_t k) { return n[k] != 0 && (counts == nullptr || counts[k] == c); };

        // ---- one launch over a device-resident plan
        size_t live = 0;
        uint64_t tiles_all = 0;
        for (size_t k = 0; k < num_tensors; ++k)
            if (member(k)) {
                ++live;
                tiles_all += (n[k] + tile - 1) / tile;
            }
        if (live == 0) continue;
        // Long lists cannot do without a plan; lists that stream 256 MiB or more per array gain
        // from one whatever their length (the plan's lookup is two scalar-cache hits where the
        // table's is a search through kernel arguments, whose latency a bandwidth-bound wave
        // feels: 64 leaves of 16 MiB run 1 to 3 % faster), and its one small fill launch per new
        // list is lost in a launch of that size.  Short lists of small tensors keep the tables.
        const bool wants_plan =
            arena != nullptr ||
            (plan_mode != 1 &&
             (plan_mode == 2 || live > (size_t)Table::MAX || tiles_all >= kPlanFromTiles));
        if (wants_plan && tiles_all < kNoTile && live < kNoTile) {
            seeds.clear();
            seeds.reserve(live);
            uint32_t first = 0;
            for (size_t k = 0; k < num_tensors; ++k) {
                if (!member(k)) continue;
                PlanSeed<Op::NPTR> seed;
                for (int i = 0; i < Op::NPTR; ++i) seed.p[i] = const_cast<void *>(lists[i][k]);
                seed.n = n[k];
                seed.first = first;
                first += (uint32_t)((n[k] + tile - 1) / tile);
                seed.next_first = first;
                seeds.push_back(seed);
            }
            const uint32_t total = (uint32_t)tiles_all;
            // the lookup is two scalar-cache hits, so a plain launch wants the residency level of
            // the single-tensor kernel, not the table kernel's raised one; a staged launch takes
            // the op's level for staged lists
            const unsigned lds = lds_reservation<Op>(staged, total, staged);
            auto launch_over = [&](void *mem, PlanView *view_out) -> int {
                const PlanView view = plan_view<Op::NPTR>(mem, seeds, total);
                if (staged) {
                    if constexpr (IsStaged<Op>::value)
                        hipLaunchKernelGGL((plan_stream_kernel<T, Op, kUnroll, kNonTemporal, true>),
                                           dim3(grid_for(total)), dim3(kBlock), lds,
                                           (hipStream_t)stream, op, view);
                } else {
                    hipLaunchKernelGGL((plan_stream_kernel<T, Op, kUnroll, kNonTemporal>),
                                       dim3(grid_for(total)), dim3(kBlock), lds,
                                       (hipStream_t)stream, op, view);
                }
                if (view_out != nullptr) *view_out = view;
                return (int)hipGetLastError();
            };
            if (arena != nullptr) {
                uint32_t fine_shift = 0;
                const uint32_t fine_entries = plan_fine_entries(live, tiles_all, &fine_shift);
                if (plan_bytes(live, fine_entries) > arena->bytes) return TOA_ELIMIT;
                if (const int rc = plan_write_all<Op::NPTR>(arena->mem, seeds, fine_entries,
                                                            fine_shift, (hipStream_t)stream))
                    return rc;
                if (const int rc = launch_over(arena->mem, nullptr)) return rc;
                continue;
            }
            int device = 0;
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            // a captured launch must not lean on memory a later call may rewrite
            const bool may_cache =
                hipStreamIsCapturing((hipStream_t)stream, &capturing) == hipSuccess &&
                capturing == hipStreamCaptureStatusNone && hipGetDevice(&device) == hipSuccess;
            if (!may_cache) (void)hipGetLastError();
            if (may_cache) {
                // lookup, rewrite and the launch that reads the plan: one step under the cache's
                // mutex (plan_cache.hpp)
                std::lock_guard<std::mutex> lock(g_plans.mutex());
                int rc = 0;
                Plans::Slot *slot =
                    plan_cached<Op::NPTR>(seeds, tile, device, (hipStream_t)stream, &rc);
                if (rc) return rc;
                if (slot != nullptr) {
                    PlanMemo memo;
                    memo.staged = staged;
                    if ((rc = launch_over(slot->mem, &memo.view)) != 0) return rc;
                    if (!call.empty()) g_plans.remember(slot, std::move(call), memo);
                    continue;
                }
            }
        } else if (arena != nullptr) {
            return TOA_ESIZE;
        }

        // ---- tables in kernel arguments, one launch each
        reset();
        auto flush = [&]() -> int {
            if (num == 0) return 0;
            tab.total = next_tile;
            if (staged) {
                if constexpr (IsStaged<Op>::value)
                    hipLaunchKernelGGL((multi_stream_kernel<T, Op, kUnroll, kNonTemporal, true>),
                                       dim3(grid_for(next_tile)), dim3(kBlock),
                                       lds_reservation<Op>(true, next_tile, true),
                                       (hipStream_t)stream, op, tab);
            } else {
                hipLaunchKernelGGL((multi_stream_kernel<T, Op, kUnroll, kNonTemporal>),
                                   dim3(grid_for(next_tile)), dim3(kBlock),
                                   lds_reservation<Op>(true, next_tile), (hipStream_t)stream, op,
                                   tab);
            }
            reset();
            return (int)hipGetLastError();
        };
        for (size_t k = 0; k < num_tensors; ++k) {
            if (!member(k)) continue;
            const uint64_t tiles = (n[k] + tile - 1) / tile;
            if (num == (uint32_t)Table::MAX || (uint64_t)next_tile + tiles >= kNoTile) {
                if (int rc = flush()) return rc;
            }
            for (int i = 0; i < Op::NPTR; ++i)
                tab.rec[num].p[i] = static_cast<T *>(const_cast<void *>(lists[i][k]));
            tab.rec[num].n = n[k];
            tab.group[num / kGroup].start[num % kGroup] = next_tile;
            if (num % kGroup == 0 && num > 0) tab.coarse[num / kGroup - 1] = next_tile;
            next_tile += (uint32_t)tiles;
            ++num;
        }
        if (int rc = flush()) return rc;
    }
    return 0;
}

// ---------------------------------------------------------------------------
// Plan memory that needs no allocation: a file-scope device array, one copy per GPU, held until
// the process ends.  Its name is a host-side stand-in, not a device address: hipGetSymbolAddress
// gives the address of the current device's copy, once per device.
// ---------------------------------------------------------------------------
constexpr size_t kNoAllocMaxTensors = 4096;
constexpr size_t kNoAllocScratchBytes =
    kNoAllocMaxTensors * sizeof(PlanRec) + 4 * kNoAllocMaxTensors * sizeof(uint32_t);  // 448 KiB
static_assert(kNoAllocScratchBytes == toa_noalloc_scratch_bytes,
              "the array holds every record and the finer index of the longest list");
constexpr int kNoAllocMaxDevices = 64;

}  // namespace

// No device code names the array (kernels receive its address as an argument); the compiler keeps
// it, with a symbol the runtime can find, because host code names it below.  (Marking it `used`
// would pin it to a local symbol, which hipGetSymbolAddress cannot resolve.)
static __device__ __align__(256) unsigned char scratch[toa_noalloc_scratch_bytes];

namespace {

std::mutex g_scratch_mutex;
void *g_scratch_ptr[kNoAllocMaxDevices] = {};

// The current device's copy of `scratch`; looked up on the first call on that device.
int scratch_for_current_device(void **out) {
    int device = 0;
    if (const int rc = (int)hipGetDevice(&device)) return rc;
    if (device < 0 || device >= kNoAllocMaxDevices) return TOA_ELIMIT;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        void *ptr = nullptr;
        if (const int rc = (int)hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) return rc;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return 0;
}

template <typename T>
T *mut(const void *p) {
    return static_cast<T *>(const_cast<void *>(p));
}

bool is_16_bit(int dtype) { return dtype == TOA_F16 || dtype == TOA_BF16; }

#define CPP(x) reinterpret_cast<const void *const *>(x)

// Calls f with two std::bool_constant tags for the run-time flags.
template <class F>
int with_flags(bool dm, bool dv, F f) {
    if (dm) return dv ? f(std::true_type{}, std::true_type{}) : f(std::true_type{}, std::false_type{});
    return dv ? f(std::false_type{}, std::true_type{}) : f(std::false_type{}, std::false_type{});
}

template <typename T, bool HAS_DM, bool HAS_DV>
int backward_all_single(const void *dnew_updates, const void *new_updates, const void *new_mu,
                        const void *updates, const void *dnew_mu, const void *dnew_nu, size_t n,
                        double b1, double b2, const HostScalars &s, void *dupdates, void *dmu,
                        void *dnu, void *stream) {
    using Op = BackwardAll<T, HAS_DM, HAS_DV>;
    const Op op{(T)b1, (T)b2, (T)s.p1, (T)s.q2};
    T *p[Op::NPTR];
    int k = 0;
    p[k++] = mut<T>(dnew_updates);
    p[k++] = mut<T>(new_updates);
    p[k++] = mut<T>(new_mu);
    p[k++] = mut<T>(updates);
    if (HAS_DM) p[k++] = mut<T>(dnew_mu);
    if (HAS_DV) p[k++] = mut<T>(dnew_nu);
    p[k++] = (T *)dupdates;
    p[k++] = (T *)dmu;
    p[k++] = (T *)dnu;
    T *const(&cp)[Op::NPTR] = p;
    return launch_single<T>(op, cp, n, stream);
}

template <typename T, bool HAS_DM, bool HAS_DV>
int backward_all_multi(size_t num, const void *const *dnew_updates,
                       const void *const *new_updates, const void *const *new_mu,
                       const void *const *updates, const void *const *dnew_mu,
                       const void *const *dnew_nu, const size_t *n, double b1, double b2,
                       double eps_root, const uint64_t *counts, uint64_t count_all,
                       void *const *dupdates, void *const *dmu, void *const *dnu, void *stream) {
    using Op = BackwardAll<T, HAS_DM, HAS_DV>;
    const void *const *lists[Op::NPTR];
    int k = 0;
    lists[k++] = dnew_updates;
    lists[k++] = new_updates;
    lists[k++] = new_mu;
    lists[k++] = updates;
    if (HAS_DM) lists[k++] = dnew_mu;
    if (HAS_DV) lists[k++] = dnew_nu;
    lists[k++] = CPP(dupdates);
    lists[k++] = CPP(dmu);
    lists[k++] = CPP(dnu);
    const void *const *const(&cl)[Op::NPTR] = lists;
    auto make = [&](uint64_t c) {
        const HostScalars s = host_scalars(b1, b2, eps_root, c);
        return Op{(T)b1, (T)b2, (T)s.p1, (T)s.q2};
    };
    return launch_multi<T, Op>(make, num, cl, n, counts, count_all, stream);
}

// every element type the reference CPU op serves
#define TOA_DISPATCH_ALL(dtype, ...)              \
    switch (dtype) {                              \
        case TOA_F32: {                           \
            using T = float;                      \
            return __VA_ARGS__();                 \
        }                                         \
        case TOA_F64: {                           \
            using T = double;                     \
            return __VA_ARGS__();                 \
        }                                         \
        case TOA_F16: {                           \
            using T = half_t;                     \
            return __VA_ARGS__();                 \
        }                                         \
        case TOA_BF16: {                          \
            using T = bfloat_t;                   \
            return __VA_ARGS__();                 \
        }                                         \
        default:                                  \
            return TOA_EDTYPE;                    \
    }

}  // namespace

extern "C" {

int toa_adam_abi_version(void) { return 5; }

// Preferred placement of state arrays: the two moments of a tensor 8 KiB apart modulo 16 KiB.
size_t toa_adam_state_slack(void) { return kStatePeriod; }

size_t toa_adam_state_shift(const void *allocation, int moment) {
    const uintptr_t want = moment == 0 ? kStatePhase : 0;
    const uintptr_t at = reinterpret_cast<uintptr_t>(allocation) % kStatePeriod;
    return (size_t)((want + kStatePeriod - at) % kStatePeriod);
}

int toa_adam_set_waves_per_cu(int waves) {
    const int prev = waves_override();
    g_waves_override.store(waves >= kMinWavesPerCU && waves <= kMaxWavesPerCU ? waves : 0,
                           std::memory_order_relaxed);
    return prev;
}

int toa_adam_set_schedule(int schedule) {
    const int prev = g_schedule.load(std::memory_order_relaxed);
    g_schedule.store(schedule == 1 || schedule == 2 ? schedule : 0, std::memory_order_relaxed);
    return prev;
}

int toa_adam_set_load_order(int order) {
    const int prev = g_load_order.load(std::memory_order_relaxed);
    g_load_order.store(order >= 0 && order <= 3 ? order : -1, std::memory_order_relaxed);
    return prev;
}

int toa_adam_set_tuning(int on) {
    const int prev = tuning_on() ? 1 : 0;
    g_tuning.store(on ? 1 : 0, std::memory_order_relaxed);
    return prev;
}

int toa_adam_tuned_load_order(int dtype, const void *updates, const void *mu, const void *nu,
                              size_t n) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    const uintptr_t p[3] = {reinterpret_cast<uintptr_t>(updates), reinterpret_cast<uintptr_t>(mu),
                            reinterpret_cast<uintptr_t>(nu)};
    auto look = [&](const void *tag, size_t tile) {
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        TuneSite *site = tune_find(tag, p, n / tile, device, false);
        if (site == nullptr) return -1;
        if (site->decided < 0) tune_collect(*site);
        return site->decided;
    };
    switch (dtype) {
        case TOA_F32: return look(&OpTag<ForwardInplace<float>>::tag, Tile<float, kUnroll>::ELEMS);
        case TOA_F64: return look(&OpTag<ForwardInplace<double>>::tag, Tile<double, kUnroll>::ELEMS);
        default: return -1;
    }
}

int toa_adam_clock_probe(uint64_t *out, uint32_t spins, void *stream) {
    if (out == nullptr) return TOA_ENULL;
    if (spins > (1u << 28)) return TOA_ESIZE;  // bounded: a few hundred milliseconds at most
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out, spins);
    return (int)hipGetLastError();
}

int toa_adam_set_plan_mode(int mode) {
    const int prev = g_plan_mode.load(std::memory_order_relaxed);
    g_plan_mode.store(mode == 1 || mode == 2 ? mode : 0, std::memory_order_relaxed);
    return prev;
}

int toa_adam_release_plans(void) {
    std::lock_guard<std::mutex> lock(g_plans.mutex());
    g_plans.release_all();
    const int rc = (int)hipGetLastError();
    return rc;
}

unsigned toa_adam_set_max_grid(unsigned workgroups) {
    const unsigned prev = g_max_grid.load(std::memory_order_relaxed);
    g_max_grid.store(workgroups >= 1 && workgroups <= kMaxGrid ? workgroups : kMaxGrid,
                     std::memory_order_relaxed);
    return prev;
}

const char *toa_adam_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case TOA_EDTYPE:
            return "toa_adam: unsupported dtype for this entry point (the fused step takes weight "
                   "decay for float32 and float64 only)";
        case TOA_ENULL: return "toa_adam: null pointer for a non-empty tensor";
        case TOA_ESIZE: return "toa_adam: tensor too large for one launch";
        case TOA_ELIMIT:
            return "toa_adam: more than 4096 non-empty tensors (or a device number beyond 63) in "
                   "a call to the allocation-free entry point";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "toa_adam: unknown error";
    }
}

int toa_adam_forward_inplace(int dtype, void *updates, void *mu, void *nu, size_t n, double b1,
                             double b2, double eps, double eps_root, uint64_t count,
                             void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    TOA_DISPATCH_ALL(dtype, [&] {
        const ForwardInplace<T> op{(T)b1, (T)b2, (T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        T *const p[3] = {(T *)updates, (T *)mu, (T *)nu};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_forward_mu(int dtype, const void *updates, const void *mu, size_t n, double b1,
                        void *mu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const ForwardMu<T> op{(T)b1};
        T *const p[3] = {mut<T>(updates), mut<T>(mu), (T *)mu_out};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_forward_nu(int dtype, const void *updates, const void *nu, size_t n, double b2,
                        void *nu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const ForwardNu<T> op{(T)b2};
        T *const p[3] = {mut<T>(updates), mut<T>(nu), (T *)nu_out};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_forward_updates(int dtype, const void *new_mu, const void *new_nu, size_t n,
                             double b1, double b2, double eps, double eps_root, uint64_t count,
                             void *updates_out, void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    TOA_DISPATCH_ALL(dtype, [&] {
        const ForwardUpdates<T> op{(T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        T *const p[3] = {mut<T>(new_mu), mut<T>(new_nu), (T *)updates_out};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_backward_mu(int dtype, const void *dmu, size_t n, double b1, void *dupdates_out,
                         void *dmu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const BackwardMu<T> op{(T)b1};
        T *const p[3] = {mut<T>(dmu), (T *)dupdates_out, (T *)dmu_out};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_backward_nu(int dtype, const void *dnu, const void *updates, size_t n, double b2,
                         void *dupdates_out, void *dnu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const BackwardNu<T> op{(T)b2};
        T *const p[4] = {mut<T>(dnu), mut<T>(updates), (T *)dupdates_out, (T *)dnu_out};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_backward_updates(int dtype, const void *dupdates, const void *updates,
                              const void *new_mu, size_t n, double b1, double b2,
                              double eps_root, uint64_t count, void *dnew_mu_out,
                              void *dnew_nu_out, void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    TOA_DISPATCH_ALL(dtype, [&] {
        const BackwardUpdates<T> op{(T)s.p1, (T)s.q2};
        T *const p[5] = {mut<T>(dupdates), mut<T>(updates), mut<T>(new_mu), (T *)dnew_mu_out,
                         (T *)dnew_nu_out};
        return launch_single<T>(op, p, n, stream);
    });
}

// ---- multi-tensor -----------------------------------------------------------


int toa_adam_forward_inplace_multi(int dtype, size_t num_tensors, void *const *updates,
                                   void *const *mu, void *const *nu, const size_t *n, double b1,
                                   double b2, double eps, double eps_root,
                                   const uint64_t *counts, uint64_t count_all, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {CPP(updates), CPP(mu), CPP(nu)};
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return ForwardInplace<T>{(T)b1, (T)b2, (T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        };
        return launch_multi<T, ForwardInplace<T>>(make, num_tensors, lists, n, counts, count_all,
                                                  stream);
    });
}

int toa_adam_forward_inplace_multi_noalloc(int dtype, size_t num_tensors, void *const *updates,
                                           void *const *mu, void *const *nu, const size_t *n,
                                           double b1, double b2, double eps, double eps_root,
                                           const uint64_t *counts, uint64_t count_all,
                                           void *stream) {
    size_t live = 0;
    if (n != nullptr)
        for (size_t k = 0; k < num_tensors; ++k) live += n[k] != 0;
    if (live > kNoAllocMaxTensors) return TOA_ELIMIT;
    PlanArena arena;
    if (live != 0) {
        if (const int rc = scratch_for_current_device(&arena.mem)) return rc;
        arena.bytes = kNoAllocScratchBytes;
    }
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {CPP(updates), CPP(mu), CPP(nu)};
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return ForwardInplace<T>{(T)b1, (T)b2, (T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        };
        return launch_multi<T, ForwardInplace<T>>(make, num_tensors, lists, n, counts, count_all,
                                                  stream, live != 0 ? &arena : nullptr);
    });
}

int toa_adam_forward_mu_multi(int dtype, size_t num_tensors, const void *const *updates,
                              const void *const *mu, const size_t *n, double b1,
                              void *const *mu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {updates, mu, CPP(mu_out)};
        auto make = [&](uint64_t) { return ForwardMu<T>{(T)b1}; };
        return launch_multi<T, ForwardMu<T>>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

int toa_adam_forward_nu_multi(int dtype, size_t num_tensors, const void *const *updates,
                              const void *const *nu, const size_t *n, double b2,
                              void *const *nu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {updates, nu, CPP(nu_out)};
        auto make = [&](uint64_t) { return ForwardNu<T>{(T)b2}; };
        return launch_multi<T, ForwardNu<T>>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

int toa_adam_forward_updates_multi(int dtype, size_t num_tensors, const void *const *new_mu,
                                   const void *const *new_nu, const size_t *n, double b1,
                                   double b2, double eps, double eps_root,
                                   const uint64_t *counts, uint64_t count_all,
                                   void *const *updates_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {new_mu, new_nu, CPP(updates_out)};
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return ForwardUpdates<T>{(T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        };
        return launch_multi<T, ForwardUpdates<T>>(make, num_tensors, lists, n, counts, count_all,
                                                  stream);
    });
}

int toa_adam_backward_mu_multi(int dtype, size_t num_tensors, const void *const *dmu,
                               const size_t *n, double b1, void *const *dupdates_out,
                               void *const *dmu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[3] = {dmu, CPP(dupdates_out), CPP(dmu_out)};
        auto make = [&](uint64_t) { return BackwardMu<T>{(T)b1}; };
        return launch_multi<T, BackwardMu<T>>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

int toa_adam_backward_nu_multi(int dtype, size_t num_tensors, const void *const *dnu,
                               const void *const *updates, const size_t *n, double b2,
                               void *const *dupdates_out, void *const *dnu_out, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[4] = {dnu, updates, CPP(dupdates_out), CPP(dnu_out)};
        auto make = [&](uint64_t) { return BackwardNu<T>{(T)b2}; };
        return launch_multi<T, BackwardNu<T>>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

int toa_adam_backward_updates_multi(int dtype, size_t num_tensors, const void *const *dupdates,
                                    const void *const *updates, const void *const *new_mu,
                                    const size_t *n, double b1, double b2, double eps_root,
                                    const uint64_t *counts, uint64_t count_all,
                                    void *const *dnew_mu_out, void *const *dnew_nu_out,
                                    void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[5] = {dupdates, updates, new_mu, CPP(dnew_mu_out),
                                             CPP(dnew_nu_out)};
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return BackwardUpdates<T>{(T)s.p1, (T)s.q2};
        };
        return launch_multi<T, BackwardUpdates<T>>(make, num_tensors, lists, n, counts,
                                                   count_all, stream);
    });
}

// ---- whole differentiable step: forward in one pass, backward in one pass -------------------

int toa_adam_forward_all(int dtype, const void *updates, const void *mu, const void *nu, size_t n,
                         double b1, double b2, double eps, double eps_root, uint64_t count,
                         void *new_mu, void *new_nu, void *new_updates, void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    TOA_DISPATCH_ALL(dtype, [&] {
        const ForwardAll<T> op{(T)b1, (T)b2, (T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        T *const p[6] = {mut<T>(updates), mut<T>(mu), mut<T>(nu),
                         (T *)new_mu,     (T *)new_nu, (T *)new_updates};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_forward_all_multi(int dtype, size_t num_tensors, const void *const *updates,
                               const void *const *mu, const void *const *nu, const size_t *n,
                               double b1, double b2, double eps, double eps_root,
                               const uint64_t *counts, uint64_t count_all, void *const *new_mu,
                               void *const *new_nu, void *const *new_updates, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[6] = {updates,     mu,          nu,
                                             CPP(new_mu), CPP(new_nu), CPP(new_updates)};
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return ForwardAll<T>{(T)b1, (T)b2, (T)s.c1, (T)s.c2, (T)eps, (T)eps_root};
        };
        return launch_multi<T, ForwardAll<T>>(make, num_tensors, lists, n, counts, count_all,
                                              stream);
    });
}

int toa_adam_backward_all(int dtype, const void *dnew_updates, const void *new_updates,
                          const void *new_mu, const void *updates, const void *dnew_mu,
                          const void *dnew_nu, size_t n, double b1, double b2, double eps_root,
                          uint64_t count, void *dupdates, void *dmu, void *dnu, void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    const bool dm = dnew_mu != nullptr, dv = dnew_nu != nullptr;
    TOA_DISPATCH_ALL(dtype, [&] {
        return with_flags(dm, dv, [&](auto DM, auto DV) {
            return backward_all_single<T, decltype(DM)::value, decltype(DV)::value>(
                dnew_updates, new_updates, new_mu, updates, dnew_mu, dnew_nu, n, b1, b2, s,
                dupdates, dmu, dnu, stream);
        });
    });
}

int toa_adam_backward_all_multi(int dtype, size_t num_tensors, const void *const *dnew_updates,
                                const void *const *new_updates, const void *const *new_mu,
                                const void *const *updates, const void *const *dnew_mu,
                                const void *const *dnew_nu, const size_t *n, double b1,
                                double b2, double eps_root, const uint64_t *counts,
                                uint64_t count_all, void *const *dupdates, void *const *dmu,
                                void *const *dnu, void *stream) {
    const bool dm = dnew_mu != nullptr, dv = dnew_nu != nullptr;
    TOA_DISPATCH_ALL(dtype, [&] {
        return with_flags(dm, dv, [&](auto DM, auto DV) {
            return backward_all_multi<T, decltype(DM)::value, decltype(DV)::value>(
                num_tensors, dnew_updates, new_updates, new_mu, updates, dnew_mu, dnew_nu, n, b1,
                b2, eps_root, counts, count_all, dupdates, dmu, dnu, stream);
        });
    });
}

// ---- fused optimizer step ------------------------------------------------------
// All four element types without weight decay; with it, float32 and float64 only: the chain the
// step reproduces applies decay with Tensor.add_(p, alpha=wd), which on 16-bit CPU tensors is not
// one arithmetic (its vectorized body and its scalar tails round differently), so there is no
// result to be identical to.

int toa_adam_fused_step(int dtype, void *params, void *updates, void *mu, void *nu, size_t n,
                        double b1, double b2, double eps, double eps_root, uint64_t count,
                        double lr, double weight_decay, int decoupled, int maximize,
                        int write_updates, void *stream) {
    const HostScalars s = host_scalars(b1, b2, eps_root, count);
    const int decay = weight_decay == 0.0 ? kNoDecay
                                          : (decoupled ? kDecayIntoUpdate : kDecayIntoGradient);
    if (decay != kNoDecay && is_16_bit(dtype)) return TOA_EDTYPE;
    TOA_DISPATCH_ALL(dtype, [&] {
        T *const p[4] = {(T *)updates, (T *)mu, (T *)nu, (T *)params};
        if (write_updates) {
            const FusedStep<T, true> op{(T)b1,       (T)b2,    (T)s.c1,         (T)s.c2, (T)eps,
                                        (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,   maximize != 0};
            return launch_single<T>(op, p, n, stream);
        }
        const FusedStep<T, false> op{(T)b1,       (T)b2,    (T)s.c1,         (T)s.c2, (T)eps,
                                     (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,   maximize != 0};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_fused_step_multi(int dtype, size_t num_tensors, void *const *params,
                              void *const *updates, void *const *mu, void *const *nu,
                              const size_t *n, double b1, double b2, double eps, double eps_root,
                              const uint64_t *counts, uint64_t count_all, double lr,
                              double weight_decay, int decoupled, int maximize,
                              int write_updates, void *stream) {
    const int decay = weight_decay == 0.0 ? kNoDecay
                                          : (decoupled ? kDecayIntoUpdate : kDecayIntoGradient);
    if (decay != kNoDecay && is_16_bit(dtype)) return TOA_EDTYPE;
    TOA_DISPATCH_ALL(dtype, [&] {
        const void *const *const lists[4] = {CPP(updates), CPP(mu), CPP(nu), CPP(params)};
        if (write_updates) {
            auto make = [&](uint64_t c) {
                const HostScalars s = host_scalars(b1, b2, eps_root, c);
                return FusedStep<T, true>{(T)b1,       (T)b2,    (T)s.c1,         (T)s.c2, (T)eps,
                                          (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,
                                          maximize != 0};
            };
            return launch_multi<T, FusedStep<T, true>>(make, num_tensors, lists, n, counts,
                                                       count_all, stream);
        }
        auto make = [&](uint64_t c) {
            const HostScalars s = host_scalars(b1, b2, eps_root, c);
            return FusedStep<T, false>{(T)b1,       (T)b2,    (T)s.c1,         (T)s.c2, (T)eps,
                                       (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,
                                       maximize != 0};
        };
        return launch_multi<T, FusedStep<T, false>>(make, num_tensors, lists, n, counts,
                                                    count_all, stream);
    });
}

// ---- step number on the device ------------------------------------------------------

int toa_adam_bias_rows(int dtype, double b1, double b2, double eps_root, uint64_t first_count,
                       size_t rows, void *host_out) {
    if (host_out == nullptr && rows != 0) return TOA_ENULL;
    TOA_DISPATCH_ALL(dtype, [&] {
        T *out = static_cast<T *>(host_out);
        for (size_t r = 0; r < rows; ++r) {
            const HostScalars s = host_scalars(b1, b2, eps_root, first_count + r);
            out[4 * r + 0] = (T)s.c1;
            out[4 * r + 1] = (T)s.c2;
            out[4 * r + 2] = (T)s.p1;
            out[4 * r + 3] = (T)s.q2;
        }
        return 0;
    });
}

size_t toa_adam_bias_rows_needed(double b1, double b2, uint64_t first_count, size_t limit) {
    // Smallest step number from which 1 - b^count is 1 in double for both decay rates: the rows
    // of every later step equal that step's.  b^count falls with count, so bisect.
    auto settled = [&](uint64_t c) {
        return 1 - std::pow(b1, (double)c) == 1.0 && 1 - std::pow(b2, (double)c) == 1.0;
    };
    if (limit == 0) return 0;
    const uint64_t hi_count = first_count + (limit - 1);
    if (!settled(hi_count)) return 0;
    uint64_t lo = first_count, hi = hi_count;  // settled(hi) holds
    while (lo < hi) {
        const uint64_t mid = lo + (hi - lo) / 2;
        if (settled(mid))
            hi = mid;
        else
            lo = mid + 1;
    }
    return (size_t)(lo - first_count + 1);
}

int toa_adam_count_advance(int64_t *count, void *stream) {
    if (count == nullptr) return TOA_ENULL;
    hipLaunchKernelGGL(count_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, count);
    return (int)hipGetLastError();
}

int toa_adam_forward_inplace_devcount(int dtype, void *updates, void *mu, void *nu, size_t n,
                                      double b1, double b2, double eps, double eps_root,
                                      const void *bias_rows, uint64_t first_count, size_t rows,
                                      const int64_t *count, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        StepRef<T> step;
        if (const int rc = make_step_ref<T>(bias_rows, first_count, rows, count, &step)) return rc;
        using Op = AtStep<ForwardInplace<T>, T>;
        const Op op{{{(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root}}, step};
        T *const p[3] = {(T *)updates, (T *)mu, (T *)nu};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_forward_inplace_multi_devcount(int dtype, size_t num_tensors, void *const *updates,
                                            void *const *mu, void *const *nu, const size_t *n,
                                            double b1, double b2, double eps, double eps_root,
                                            const void *bias_rows, uint64_t first_count,
                                            size_t rows, const int64_t *count, void *stream) {
    TOA_DISPATCH_ALL(dtype, [&] {
        StepRef<T> step;
        if (const int rc = make_step_ref<T>(bias_rows, first_count, rows, count, &step)) return rc;
        using Op = AtStep<ForwardInplace<T>, T>;
        const void *const *const lists[3] = {CPP(updates), CPP(mu), CPP(nu)};
        auto make = [&](uint64_t) {
            return Op{{{(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root}}, step};
        };
        return launch_multi<T, Op>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

int toa_adam_fused_step_devcount(int dtype, void *params, void *updates, void *mu, void *nu,
                                 size_t n, double b1, double b2, double eps, double eps_root,
                                 const void *bias_rows, uint64_t first_count, size_t rows,
                                 const int64_t *count, double lr, double weight_decay,
                                 int decoupled, int maximize, int write_updates, void *stream) {
    const int decay = weight_decay == 0.0 ? kNoDecay
                                          : (decoupled ? kDecayIntoUpdate : kDecayIntoGradient);
    if (decay != kNoDecay && is_16_bit(dtype)) return TOA_EDTYPE;
    TOA_DISPATCH_ALL(dtype, [&] {
        StepRef<T> step;
        if (const int rc = make_step_ref<T>(bias_rows, first_count, rows, count, &step)) return rc;
        T *const p[4] = {(T *)updates, (T *)mu, (T *)nu, (T *)params};
        if (write_updates) {
            const AtStep<FusedStep<T, true>, T> op{
                {(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,
                 maximize != 0},
                step};
            return launch_single<T>(op, p, n, stream);
        }
        const AtStep<FusedStep<T, false>, T> op{
            {(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay, decay,
             maximize != 0},
            step};
        return launch_single<T>(op, p, n, stream);
    });
}

int toa_adam_fused_step_multi_devcount(int dtype, size_t num_tensors, void *const *params,
                                       void *const *updates, void *const *mu, void *const *nu,
                                       const size_t *n, double b1, double b2, double eps,
                                       double eps_root, const void *bias_rows,
                                       uint64_t first_count, size_t rows, const int64_t *count,
                                       double lr, double weight_decay, int decoupled,
                                       int maximize, int write_updates, void *stream) {
    const int decay = weight_decay == 0.0 ? kNoDecay
                                          : (decoupled ? kDecayIntoUpdate : kDecayIntoGradient);
    if (decay != kNoDecay && is_16_bit(dtype)) return TOA_EDTYPE;
    TOA_DISPATCH_ALL(dtype, [&] {
        StepRef<T> step;
        if (const int rc = make_step_ref<T>(bias_rows, first_count, rows, count, &step)) return rc;
        const void *const *const lists[4] = {CPP(updates), CPP(mu), CPP(nu), CPP(params)};
        if (write_updates) {
            using Op = AtStep<FusedStep<T, true>, T>;
            auto make = [&](uint64_t) {
                return Op{{(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root, (StepScalar<T>)(-lr),
                           (StepScalar<T>)weight_decay, decay, maximize != 0},
                          step};
            };
            return launch_multi<T, Op>(make, num_tensors, lists, n, nullptr, 0, stream);
        }
        using Op = AtStep<FusedStep<T, false>, T>;
        auto make = [&](uint64_t) {
            return Op{{(T)b1, (T)b2, T(1), T(1), (T)eps, (T)eps_root, (StepScalar<T>)(-lr), (StepScalar<T>)weight_decay,
                       decay, maximize != 0},
                      step};
        };
        return launch_multi<T, Op>(make, num_tensors, lists, n, nullptr, 0, stream);
    });
}

}  // extern "C"
