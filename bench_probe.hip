// Memory-system probes for bench.py --ceiling: streaming kernels with next to no arithmetic.
// They measure what this machine's HBM delivers (a) for R arrays read and W arrays written per
// pass with the launch shape of the Adam kernels, and (b) for the in-place step's pattern --
// three arrays read and written back -- under a FAMILY of launch shapes and two array layouts,
// so that the ceiling quoted beside the operator is the machine's and not one kernel shape's.
// Measurement tool only: nothing in the library or the package uses it.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kWave = 64;
constexpr int kMaxArrays = 9;

#define PROBE_LD(p) __builtin_nontemporal_load(p)
#define PROBE_ST(v, p) __builtin_nontemporal_store(v, p)
#define PROBE_WAIT() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")

struct Arrays {
    f4 *p[kMaxArrays];  // reads first, then writes
};

template <int R, int W>
__global__ __launch_bounds__(kWave) void probe_kernel(Arrays a, size_t vecs) {
    const size_t i = (size_t)blockIdx.x * kWave + threadIdx.x;
    if (i >= vecs) return;
    f4 acc = {1.0f, 2.0f, 3.0f, 4.0f};
#pragma unroll
    for (int r = 0; r < R; ++r) acc += PROBE_LD(a.p[r] + i);
    if constexpr (W == 0) {
        // keeps the loads alive; the inputs are never this value, so nothing is written
        if (acc.x == 123456.78125f) a.p[0][i] = acc;
    } else {
#pragma unroll
        for (int w = 0; w < W; ++w) PROBE_ST(acc + (float)w, a.p[R + w] + i);
    }
}

template <int R, int W>
int launch(void *const *ptrs, size_t bytes, unsigned lds, hipStream_t stream) {
    Arrays a{};
    for (int k = 0; k < R + W; ++k) a.p[k] = (f4 *)ptrs[k];
    const size_t vecs = bytes / sizeof(f4);
    const size_t grid = (vecs + kWave - 1) / kWave;
    if (grid == 0 || grid > 0x7fffffffu) return -3;
    hipLaunchKernelGGL((probe_kernel<R, W>), dim3((unsigned)grid), dim3(kWave), lds, stream, a,
                       vecs);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Three arrays read and written back, under a family of launch shapes.
//
// Layout of the three arrays: three separate allocations (piece == 0: vector i of array k is
// base[k] + i), or one arena in which they interleave in pieces of `piece` vectors (vector i of
// array k is base[0] + ((i / piece) * 3 + k) * piece + i % piece) -- the same bytes, the same
// access pattern per array, another placement in DRAM.
// ---------------------------------------------------------------------------
struct Three {
    f4 *base[3];
    size_t piece;  // vectors per piece, a multiple of 64; 0 = separate arrays
    __device__ __forceinline__ f4 *at(int k, size_t i) const {
        return piece == 0 ? base[k] + i : base[0] + ((i / piece) * 3 + k) * piece + i % piece;
    }
};

// What is written back is what was read, rotated between the arrays (array 1 receives array 0's
// tile, 2 receives 1's, 0 receives 2's): no arithmetic, and the data stays as random as it was,
// pass after pass -- HBM throughput depends on the bits moved (a zero-filled array streams 3 %
// faster), so the probe must not smooth its data.

// one tile (1 KiB of each array) per wave; WAVES waves per workgroup, TILES tiles per wave with
// every load issued before the first store
template <int WAVES, int TILES>
__global__ __launch_bounds__(WAVES *kWave) void shape_dispatch(Three t) {
    const size_t v0 = (size_t)blockIdx.x * (WAVES * kWave * TILES) + threadIdx.x;
    f4 a[TILES], b[TILES], c[TILES];
#pragma unroll
    for (int k = 0; k < TILES; ++k) {
        const size_t i = v0 + (size_t)k * (WAVES * kWave);
        a[k] = PROBE_LD(t.at(0, i));
        b[k] = PROBE_LD(t.at(1, i));
        c[k] = PROBE_LD(t.at(2, i));
    }
#pragma unroll
    for (int k = 0; k < TILES; ++k) {
        const size_t i = v0 + (size_t)k * (WAVES * kWave);
        PROBE_ST(a[k], t.at(1, i));
        PROBE_ST(b[k], t.at(2, i));
        PROBE_ST(c[k], t.at(0, i));
    }
}

// one memory operation of the wave at a time: load | load | store, load | store, store
__global__ __launch_bounds__(kWave) void shape_staged(Three t) {
    const size_t i = (size_t)blockIdx.x * kWave + threadIdx.x;
    const f4 a = PROBE_LD(t.at(0, i));
    PROBE_WAIT();
    const f4 b = PROBE_LD(t.at(1, i));
    PROBE_WAIT();
    PROBE_ST(a, t.at(1, i));
    const f4 c = PROBE_LD(t.at(2, i));
    PROBE_WAIT();
    PROBE_ST(b, t.at(2, i));
    PROBE_ST(c, t.at(0, i));
}

// SEQ tiles per wave, one after the other, each with the staged order (a wave owns SEQ adjacent
// tiles: what a list kernel would do to spread the cost of finding its tensor over more bytes)
template <int SEQ>
__global__ __launch_bounds__(kWave) void shape_staged_seq(Three t) {
#pragma unroll 1
    for (int k = 0; k < SEQ; ++k) {
        const size_t i = ((size_t)blockIdx.x * SEQ + k) * kWave + threadIdx.x;
        const f4 a = PROBE_LD(t.at(0, i));
        PROBE_WAIT();
        const f4 b = PROBE_LD(t.at(1, i));
        PROBE_WAIT();
        PROBE_ST(a, t.at(1, i));
        const f4 c = PROBE_LD(t.at(2, i));
        PROBE_WAIT();
        PROBE_ST(b, t.at(2, i));
        PROBE_ST(c, t.at(0, i));
    }
}

// a wait after every load and every store
__global__ __launch_bounds__(kWave) void shape_serial(Three t) {
    const size_t i = (size_t)blockIdx.x * kWave + threadIdx.x;
    const f4 a = PROBE_LD(t.at(0, i));
    PROBE_WAIT();
    const f4 b = PROBE_LD(t.at(1, i));
    PROBE_WAIT();
    const f4 c = PROBE_LD(t.at(2, i));
    PROBE_WAIT();
    PROBE_ST(a, t.at(1, i));
    PROBE_WAIT();
    PROBE_ST(b, t.at(2, i));
    PROBE_WAIT();
    PROBE_ST(c, t.at(0, i));
}

// persistent grid: a wave strides over the tiles and loads its next tile before it stores the
// current one
__global__ __launch_bounds__(kWave) void shape_gridstride(Three t, unsigned tiles) {
    unsigned tile = blockIdx.x;
    if (tile >= tiles) return;
    size_t i = (size_t)tile * kWave + threadIdx.x;
    f4 a = PROBE_LD(t.at(0, i)), b = PROBE_LD(t.at(1, i)), c = PROBE_LD(t.at(2, i));
    for (;;) {
        const unsigned next = tile + gridDim.x;
        const bool more = next < tiles;
        const size_t j = (size_t)next * kWave + threadIdx.x;
        f4 a2, b2, c2;
        if (more) {
            a2 = PROBE_LD(t.at(0, j));
            b2 = PROBE_LD(t.at(1, j));
            c2 = PROBE_LD(t.at(2, j));
        }
        PROBE_ST(a, t.at(1, i));
        PROBE_ST(b, t.at(2, i));
        PROBE_ST(c, t.at(0, i));
        if (!more) break;
        a = a2, b = b2, c = c2, tile = next, i = j;
    }
}

}  // namespace

// One pass reading `reads` arrays and writing `writes` arrays of `bytes` bytes each (a multiple
// of 16), `ptrs` = device pointers, reads first.  `lds_bytes` of dynamic LDS are reserved per
// workgroup to cap residency.  Served shapes: (1,0) (3,0) (0,1) (0,3) (1,1) (2,1) (3,3) (4,3),
// and the backward ops' (1,2) (2,2) (3,2) (6,3).
extern "C" __attribute__((visibility("default"))) int bench_probe_stream(
    int reads, int writes, void *const *ptrs, size_t bytes, unsigned lds_bytes, void *stream) {
    if (ptrs == nullptr || bytes % 16 != 0) return -2;
    hipStream_t s = (hipStream_t)stream;
    switch (reads * 10 + writes) {
        case 10: return launch<1, 0>(ptrs, bytes, lds_bytes, s);
        case 30: return launch<3, 0>(ptrs, bytes, lds_bytes, s);
        case 1: return launch<0, 1>(ptrs, bytes, lds_bytes, s);
        case 3: return launch<0, 3>(ptrs, bytes, lds_bytes, s);
        case 11: return launch<1, 1>(ptrs, bytes, lds_bytes, s);
        case 21: return launch<2, 1>(ptrs, bytes, lds_bytes, s);
        case 12: return launch<1, 2>(ptrs, bytes, lds_bytes, s);
        case 22: return launch<2, 2>(ptrs, bytes, lds_bytes, s);
        case 32: return launch<3, 2>(ptrs, bytes, lds_bytes, s);
        case 63: return launch<6, 3>(ptrs, bytes, lds_bytes, s);
        case 33: return launch<3, 3>(ptrs, bytes, lds_bytes, s);
        case 43: return launch<4, 3>(ptrs, bytes, lds_bytes, s);
        default: return -1;
    }
}

// Launch shapes of bench_probe_inplace3.
enum {
    PROBE_WAVE_TILE = 0,   // 1 wave per workgroup, 1 tile per wave (the operator's plain shape)
    PROBE_STAGED = 1,      // same, one memory operation at a time (the operator's staged shape)
    PROBE_SERIAL = 2,      // same, a wait after every load and store
    PROBE_WG256 = 3,       // 4 waves per workgroup
    PROBE_WG512 = 4,       // 8 waves per workgroup
    PROBE_TILES2 = 5,      // 2 tiles per wave, loads first
    PROBE_TILES4 = 6,      // 4 tiles per wave, loads first
    PROBE_GRIDSTRIDE = 7,  // persistent grid of `param` workgroups per CU x 256 CUs, prefetching
    PROBE_STAGED_SEQ2 = 8,  // staged, two adjacent tiles per wave, one after the other
    PROBE_STAGED_SEQ4 = 9,  // staged, four adjacent tiles per wave, one after the other
    PROBE_SHAPES = 10
};

// Three arrays of `bytes` bytes each (a multiple of 4 KiB x the shape's tiles per workgroup)
// read and written back in one pass.  piece_bytes == 0: a0, a1, a2 are three arrays; otherwise
// a0 is one arena of 3 * bytes in which the arrays interleave in pieces of piece_bytes (a
// multiple of 1 KiB that divides `bytes`; a1 and a2 are ignored).  `lds_bytes` of dynamic LDS per
// workgroup cap residency; `param` is the workgroups per compute unit of PROBE_GRIDSTRIDE.
extern "C" __attribute__((visibility("default"))) int bench_probe_inplace3(
    int shape, void *a0, void *a1, void *a2, size_t bytes, size_t piece_bytes, unsigned lds_bytes,
    int param, void *stream) {
    if (a0 == nullptr || (piece_bytes == 0 && (a1 == nullptr || a2 == nullptr))) return -2;
    if (bytes == 0 || bytes % 4096 != 0 || piece_bytes % 1024 != 0 ||
        (piece_bytes != 0 && bytes % piece_bytes != 0))
        return -2;
    const Three t{{(f4 *)a0, (f4 *)a1, (f4 *)a2}, piece_bytes / sizeof(f4)};
    const size_t tiles = bytes / 1024;
    if (tiles > 0x7fffffffu) return -3;
    hipStream_t s = (hipStream_t)stream;
    auto grid = [&](size_t tiles_per_workgroup) { return dim3((unsigned)(tiles / tiles_per_workgroup)); };
    switch (shape) {
        case PROBE_WAVE_TILE:
            hipLaunchKernelGGL((shape_dispatch<1, 1>), grid(1), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_STAGED:
            hipLaunchKernelGGL(shape_staged, grid(1), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_SERIAL:
            hipLaunchKernelGGL(shape_serial, grid(1), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_WG256:
            hipLaunchKernelGGL((shape_dispatch<4, 1>), grid(4), dim3(256), lds_bytes, s, t);
            break;
        case PROBE_WG512:
            if (tiles % 8) return -2;
            hipLaunchKernelGGL((shape_dispatch<8, 1>), grid(8), dim3(512), lds_bytes, s, t);
            break;
        case PROBE_TILES2:
            hipLaunchKernelGGL((shape_dispatch<1, 2>), grid(2), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_TILES4:
            hipLaunchKernelGGL((shape_dispatch<1, 4>), grid(4), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_GRIDSTRIDE:
            if (param < 1 || param > 32) return -2;
            hipLaunchKernelGGL(shape_gridstride, dim3(256u * (unsigned)param), dim3(64), 0, s, t,
                               (unsigned)tiles);
            break;
        case PROBE_STAGED_SEQ2:
            hipLaunchKernelGGL((shape_staged_seq<2>), grid(2), dim3(64), lds_bytes, s, t);
            break;
        case PROBE_STAGED_SEQ4:
            hipLaunchKernelGGL((shape_staged_seq<4>), grid(4), dim3(64), lds_bytes, s, t);
            break;
        default:
            return -1;
    }
    return (int)hipGetLastError();
}
