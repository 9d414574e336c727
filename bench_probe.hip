// Memory-system probes for bench.py --ceiling: streaming kernels with the launch shape of the
// Adam kernels (one wavefront per workgroup, one 1 KiB tile of every array per workgroup, 128-bit
// non-temporal accesses, residency capped through a dynamic-LDS reservation) and next to no
// arithmetic.  They measure what this machine's HBM delivers for R arrays read and W arrays
// written per pass -- the ceiling the Adam kernels are compared with.  Measurement tool only:
// nothing in the library or the package uses it.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kBlock = 64;
constexpr int kMaxArrays = 8;

struct Arrays {
    f4 *p[kMaxArrays];  // reads first, then writes
};

template <int R, int W>
__global__ __launch_bounds__(kBlock) void probe_kernel(Arrays a, size_t vecs) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= vecs) return;
    f4 acc = {1.0f, 2.0f, 3.0f, 4.0f};
#pragma unroll
    for (int r = 0; r < R; ++r) acc += __builtin_nontemporal_load(a.p[r] + i);
    if constexpr (W == 0) {
        // keeps the loads alive; the inputs are never this value, so nothing is written
        if (acc.x == 123456.78125f) a.p[0][i] = acc;
    } else {
#pragma unroll
        for (int w = 0; w < W; ++w) __builtin_nontemporal_store(acc + (float)w, a.p[R + w] + i);
    }
}

template <int R, int W>
int launch(void *const *ptrs, size_t bytes, unsigned lds, hipStream_t stream) {
    Arrays a{};
    for (int k = 0; k < R + W; ++k) a.p[k] = (f4 *)ptrs[k];
    const size_t vecs = bytes / sizeof(f4);
    const size_t grid = (vecs + kBlock - 1) / kBlock;
    if (grid == 0 || grid > 0x7fffffffu) return -3;
    hipLaunchKernelGGL((probe_kernel<R, W>), dim3((unsigned)grid), dim3(kBlock), lds, stream, a,
                       vecs);
    return (int)hipGetLastError();
}

}  // namespace

// One pass reading `reads` arrays and writing `writes` arrays of `bytes` bytes each (a multiple
// of 16), `ptrs` = device pointers, reads first.  `lds_bytes` of dynamic LDS are reserved per
// workgroup to cap residency.  Served shapes: (1,0) (3,0) (0,1) (0,3) (1,1) (2,1) (3,3) (4,3).
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
        case 33: return launch<3, 3>(ptrs, bytes, lds_bytes, s);
        case 43: return launch<4, 3>(ptrs, bytes, lds_bytes, s);
        default: return -1;
    }
}
