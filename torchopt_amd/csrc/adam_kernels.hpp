// Device code of the fused Adam operator for gfx950 (MI355X, CDNA4).
//
// Every op here is a pure streaming pass: a handful of flops per element
// against 12-48 bytes of HBM traffic, so the kernels are shaped for memory
// throughput and nothing else.  What measurement on MI355X settled:
//   * 128-bit accesses (4 x f32 or 2 x f64 per lane): one wave instruction
//     covers 1 KiB of contiguous memory;
//   * a workgroup is ONE wavefront and handles ONE tile (1 KiB of every
//     stream).  The grid has one workgroup per tile, so the hardware
//     dispatcher hands out tiles in address order and the set of tiles in
//     flight is one compact window that slides through each array -- DRAM
//     pages and the TLB see a sequential stream even though thousands of
//     waves run at once.  Coarser tiles, contiguous per-workgroup chunks and
//     persistent grid-stride grids all measured 5-20 % slower on the
//     read-modify-write stream;
//   * residency is capped per op (kWavesPerCU for the single-tensor kernel,
//     kWavesPerCUMulti for the multi-tensor one, enforced through a dynamic-LDS
//     reservation made at launch): more bytes in flight than the memory
//     system needs only lengthens queues and widens the window.  LDS granules
//     make 32, 25, 21, 18, 16, 14, 12, 11, 10 ... the levels that exist; the
//     in-place step peaks at 18 waves per CU in its staged schedule (12 in the plain one), the
//     out-of-place ops at 16-32;
//   * every array is touched once, so loads and stores carry the
//     non-temporal hint (worth ~10 %);
//   * the in-place step runs a staged schedule (tile_full_staged): one memory
//     operation of a wave at a time, each result stored as soon as it exists --
//     load g | load mu | store mu', load nu | store nu', store u'.  A wave then
//     never presents the memory system with three reads (or three writes) to
//     three arrays at once.  That is worth 1.5-2 % where the arrays lie a
//     multiple of 2 MiB apart (what a caching allocator hands out for large
//     tensors) and removes a 10-17 % loss where they lie a multiple of 16 MiB
//     apart (three accesses of one wave then meet in one DRAM bank).
//
// Arithmetic follows /root/reference/src/adam_op/adam_op_impl_cpu.cpp to the
// rounding: every product and sum is rounded on its own (build with
// -ffp-contract=off), (1-b) is formed in the element type, bias corrections
// are pre-rounded reciprocals that multiply, sqrt and divide are the
// correctly rounded ones (the 16-bit types reach the same bits through a checked
// shortcut, see adam_direction_quick), and the tail of backward_updates runs in
// double.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace toa {

constexpr int kBlock = 64;  // one wavefront per workgroup

// ---------------------------------------------------------------------------
// 16-bit element types with the arithmetic of c10::Half / c10::BFloat16, which
// is what the reference CPU op computes in when it is handed such tensors
// (/root/reference/include/common.h:26-31): an operation between two 16-bit
// values (or an int, which converts first) runs in float and is rounded back to
// 16 bits; an operation with a float (double) operand yields an unrounded float
// (double); a double reaches 16 bits through float.
// ---------------------------------------------------------------------------
struct HalfFormat {  // IEEE binary16
    static __host__ __device__ inline uint16_t encode(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));  // v_cvt_f16_f32, RNE
#else
        uint32_t x = __builtin_bit_cast(uint32_t, f);
        const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
        x &= 0x7fffffffu;
        if (x > 0x7f800000u) return sign | 0x7e00u;
        if (x >= 0x477ff000u) return sign | 0x7c00u;
        if (x < 0x38800000u) {  // subnormal: count units of 2^-24, ties to even
            const float units = __builtin_bit_cast(float, x) * 16777216.0f;
            uint32_t q = (uint32_t)units;
            const float frac = units - (float)q;
            if (frac > 0.5f || (frac == 0.5f && (q & 1u))) ++q;
            return sign | (uint16_t)q;
        }
        uint32_t h = (((x >> 23) - 112u) << 10) | ((x & 0x7fffffu) >> 13);
        const uint32_t rest = x & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) ++h;
        return sign | (uint16_t)h;
#endif
    }
    // two values at once (element 0 in the low half); same rounding as encode / decode
    static __host__ __device__ inline uint32_t encode2(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        typedef float float2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, half2_t));
#else
        return (uint32_t)encode(lo) | ((uint32_t)encode(hi) << 16);
#endif
    }
    static __host__ __device__ inline void decode2(uint32_t p, float &lo, float &hi) {
        lo = decode((uint16_t)(p & 0xffffu));
        hi = decode((uint16_t)(p >> 16));
    }
    static __host__ __device__ inline void round2(float a, float b, float &lo, float &hi) {
        decode2(encode2(a, b), lo, hi);
    }
    static __host__ __device__ inline float decode(uint16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
        return static_cast<float>(__builtin_bit_cast(_Float16, h));
#else
        const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
        if (e == 0) return __builtin_bit_cast(float, sign) + (sign ? -1.0f : 1.0f) * (float)m * 5.9604644775390625e-8f;
        if (e == 31) return __builtin_bit_cast(float, sign | 0x7f800000u | (m << 13));
        return __builtin_bit_cast(float, sign | ((e + 112u) << 23) | (m << 13));
#endif
    }
};

struct BFloatFormat {  // upper half of a binary32, round to nearest even
    static __host__ __device__ inline uint16_t encode(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
        // v_cvt_pk_bf16_f32: same rounding; a NaN stays a (quiet) NaN with its own payload
        return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
#else
        const uint32_t x = __builtin_bit_cast(uint32_t, f);
        if ((x & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
        return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
#endif
    }
    static __host__ __device__ inline float decode(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    // two values at once (element 0 in the low half): one v_cvt_pk_bf16_f32 rounds both
    static __host__ __device__ inline uint32_t encode2(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __bf16 bfloat2_t __attribute__((ext_vector_type(2)));
        typedef float float2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bfloat2_t));
#else
        return (uint32_t)encode(lo) | ((uint32_t)encode(hi) << 16);
#endif
    }
    static __host__ __device__ inline void decode2(uint32_t p, float &lo, float &hi) {
        lo = __builtin_bit_cast(float, p << 16);
        hi = __builtin_bit_cast(float, p & 0xffff0000u);
    }
    // f rounded to bfloat16 and left in a float: a bfloat16 is the upper half of a float, so
    // converting the pair (0, f) yields that float's bit pattern outright -- one instruction,
    // where convert-then-widen takes two.
    static __host__ __device__ inline float rounded(float f) {
        return __builtin_bit_cast(float, encode2(0.0f, f));
    }
    static __host__ __device__ inline void round2(float a, float b, float &lo, float &hi) {
        lo = rounded(a);
        hi = rounded(b);
    }
};

template <class F>
struct R16 {
    uint16_t bits;
    R16() = default;
    __host__ __device__ R16(float f) : bits(F::encode(f)) {}
    __host__ __device__ explicit R16(double d) : bits(F::encode((float)d)) {}
    __host__ __device__ R16(int i) : bits(F::encode((float)i)) {}
    __host__ __device__ static R16 from_bits(uint16_t b) {
        R16 r;
        r.bits = b;
        return r;
    }
    __host__ __device__ operator float() const { return F::decode(bits); }
};
// A float result that is about to be rounded to 16 bits, kept apart from that rounding.  The
// reference rounds twice there -- the float operation to 24 bits, then the conversion to 16 -- and
// the compiler would merge a float16 operand's widening, the float operation and the conversion
// into ONE mixed-precision instruction (v_fma_mixlo_f16) that rounds once.  Between two 16-bit
// operands that is the same value (a product is exact in float, a sum's double rounding is
// innocuous); with a float operand of 24 significant bits (the step's -lr) it is not: 1490 x
// 2^-24 times float(-0.05) is 74.5000011 units of 2^-24, which the float product rounds to the
// tie 74.5 and the conversion to 74, where one rounding gives 75.
__host__ __device__ inline float rounded_to_float(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(x));
#endif
    return x;
}
#define TOA_R16_BINOP(OP)                                                                        \
    template <class F>                                                                           \
    __host__ __device__ inline R16<F> operator OP(R16<F> a, R16<F> b) {                          \
        return R16<F>((float)a OP(float) b);                                                     \
    }                                                                                            \
    template <class F>                                                                           \
    __host__ __device__ inline R16<F> operator OP(int a, R16<F> b) {                             \
        return R16<F>(a) OP b;                                                                   \
    }                                                                                            \
    template <class F>                                                                           \
    __host__ __device__ inline float operator OP(R16<F> a, float b) {                            \
        return rounded_to_float((float)a OP b);                                                  \
    }                                                                                            \
    template <class F>                                                                           \
    __host__ __device__ inline float operator OP(float a, R16<F> b) {                            \
        return rounded_to_float(a OP(float) b);                                                  \
    }                                                                                            \
    template <class F>                                                                           \
    __host__ __device__ inline double operator OP(R16<F> a, double b) {                          \
        return (double)(float)a OP b;                                                            \
    }                                                                                            \
    template <class F>                                                                           \
    __host__ __device__ inline double operator OP(double a, R16<F> b) {                          \
        return a OP(double)(float) b;                                                            \
    }
TOA_R16_BINOP(+)
TOA_R16_BINOP(-)
TOA_R16_BINOP(*)
TOA_R16_BINOP(/)
#undef TOA_R16_BINOP
template <class F>
__host__ __device__ inline R16<F> operator-(R16<F> a) { return R16<F>(-(float)a); }
template <class F>
__host__ __device__ inline bool operator==(R16<F> a, int b) { return (float)a == (float)b; }

using half_t = R16<HalfFormat>;
using bfloat_t = R16<BFloatFormat>;

// ---------------------------------------------------------------------------
// Two 16-bit values computed side by side (device code only).  Same arithmetic as R16 -- every
// operation between 16-bit values rounded back to 16 bits, operations with a float operand left
// unrounded -- but the two values stay in registers as floats that are exactly representable in
// the 16-bit format: a bfloat16 rounding is then ONE instruction (see BFloatFormat::rounded)
// instead of convert-and-widen, a float16 rounding one packed conversion for both values, and
// the two results leave as one packed word.  Roundings are what the 16-bit kernels spend most of
// their time on.
// ---------------------------------------------------------------------------
struct Float2 {  // two unrounded floats
    float lo, hi;
};

template <class F>
struct Pair16 {
    float lo, hi;  // each exactly representable in F
    Pair16() = default;
    __device__ static Pair16 from_bits(uint32_t p) {
        Pair16 r;
        F::decode2(p, r.lo, r.hi);
        return r;
    }
    __device__ static Pair16 rounded(float a, float b) {
        Pair16 r;
        F::round2(a, b, r.lo, r.hi);
        return r;
    }
    __device__ uint32_t bits() const { return F::encode2(lo, hi); }  // exact: nothing to round
    __device__ explicit Pair16(R16<F> s) {
        lo = hi = (float)s;
    }
    __device__ Pair16(int i) { *this = rounded((float)i, (float)i); }
    __device__ Pair16(Float2 f) { *this = rounded(f.lo, f.hi); }  // the one rounding of a result
    __device__ float low() const { return lo; }
    __device__ float high() const { return hi; }
};

// float16 pairs compute in the hardware's own packed half arithmetic.  An operation between two
// float16 values, run in float and rounded back (what c10::Half does), IS the correctly rounded
// float16 operation: a product of two 11-bit significands is exact in float's 24, and a sum or
// difference rounded first to 24 bits and then to 11 rounds as if rounded once (double rounding is
// innocuous when the wider format has at least 2 x 11 + 2 bits).  So v_pk_mul_f16 / v_pk_add_f16
// give the reference's bits for two elements per instruction with no conversion in between --
// never fused: the build contracts nothing.  The root, the sum with eps and the quotient of the
// step direction stay in float, as for one value.
template <>
struct Pair16<HalfFormat> {
    typedef _Float16 Halves __attribute__((ext_vector_type(2)));
    Halves v;
    Pair16() = default;
    __device__ static Pair16 from_bits(uint32_t p) {
        Pair16 r;
        r.v = __builtin_bit_cast(Halves, p);
        return r;
    }
    __device__ static Pair16 rounded(float a, float b) {
        // the floats are results of float operations: see rounded_to_float
        return from_bits(HalfFormat::encode2(rounded_to_float(a), rounded_to_float(b)));
    }
    __device__ uint32_t bits() const { return __builtin_bit_cast(uint32_t, v); }
    __device__ explicit Pair16(R16<HalfFormat> s) {
        // through integer arithmetic: picking a 16-bit field out of the op as a half vector makes
        // the compiler keep the op in memory (promoted to LDS, which costs residency)
        const uint32_t w = s.bits;
        v = __builtin_bit_cast(Halves, w | (w << 16));
    }
    __device__ Pair16(int i) {
        const _Float16 h = static_cast<_Float16>(static_cast<float>(i));
        v = Halves{h, h};
    }
    __device__ Pair16(Float2 f) { *this = rounded(f.lo, f.hi); }  // the one rounding of a result
    __device__ float low() const { return static_cast<float>(v[0]); }
    __device__ float high() const { return static_cast<float>(v[1]); }
};
// sums, differences and products of float16 pairs: the packed half instructions
#define TOA_HALF_PAIR_BINOP(OP)                                                                  \
    __device__ inline Pair16<HalfFormat> operator OP(Pair16<HalfFormat> a,                       \
                                                     Pair16<HalfFormat> b) {                     \
        Pair16<HalfFormat> r;                                                                    \
        r.v = a.v OP b.v;                                                                        \
        return r;                                                                                \
    }
TOA_HALF_PAIR_BINOP(+)
TOA_HALF_PAIR_BINOP(-)
TOA_HALF_PAIR_BINOP(*)
#undef TOA_HALF_PAIR_BINOP
// a quotient of float16 values goes through float's correctly rounded division
__device__ inline Pair16<HalfFormat> operator/(Pair16<HalfFormat> a, Pair16<HalfFormat> b) {
    return Pair16<HalfFormat>::rounded(a.low() / b.low(), a.high() / b.high());
}
#define TOA_PAIR_BINOP(OP)                                                                       \
    template <class F>                                                                           \
    __device__ inline Pair16<F> operator OP(Pair16<F> a, Pair16<F> b) {                          \
        return Pair16<F>::rounded(a.lo OP b.lo, a.hi OP b.hi);                                   \
    }                                                                                            \
    template <class F>                                                                           \
    __device__ inline Pair16<F> operator OP(int a, Pair16<F> b) {                                \
        return Pair16<F>(a) OP b;                                                                \
    }                                                                                            \
    __device__ inline Pair16<HalfFormat> operator OP(int a, Pair16<HalfFormat> b) {              \
        return Pair16<HalfFormat>(a) OP b;                                                       \
    }                                                                                            \
    template <class F>                                                                           \
    __device__ inline Float2 operator OP(Pair16<F> a, Float2 b) {                                \
        return {a.low() OP b.lo, a.high() OP b.hi};                                              \
    }                                                                                            \
    template <class F>                                                                           \
    __device__ inline Float2 operator OP(Float2 a, Pair16<F> b) {                                \
        return {a.lo OP b.low(), a.hi OP b.high()};                                              \
    }
TOA_PAIR_BINOP(+)
TOA_PAIR_BINOP(-)
TOA_PAIR_BINOP(*)
TOA_PAIR_BINOP(/)
#undef TOA_PAIR_BINOP
template <typename T>
struct PairOf {  // the pair type a 16-bit element type computes in; void for the wide types
    using type = void;
};
template <class F>
struct PairOf<R16<F>> {
    using type = Pair16<F>;
};

// 128-bit access types and element accessors.
template <typename T>
struct Vec;
template <>
struct Vec<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    static constexpr int N = 4;
    __device__ static float get(const type &v, int e) { return v[e]; }
    __device__ static void set(type &v, int e, float x) { v[e] = x; }
};
template <>
struct Vec<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    static constexpr int N = 2;
    __device__ static double get(const type &v, int e) { return v[e]; }
    __device__ static void set(type &v, int e, double x) { v[e] = x; }
};
template <class F>
struct Vec<R16<F>> {
    typedef uint16_t type __attribute__((ext_vector_type(8)));
    static constexpr int N = 8;
    __device__ static R16<F> get(const type &v, int e) { return R16<F>::from_bits(v[e]); }
    __device__ static void set(type &v, int e, R16<F> x) { v[e] = x.bits; }
};

// Every array these kernels touch is device memory (the entry points' contract); a pointer that
// reached the kernel through memory -- a plan's record -- carries no address space the compiler
// could see, and would be served by FLAT instructions (aperture checks, both memory counters).
// All accesses therefore go through the global address space explicitly.
template <typename V>
__device__ __forceinline__ auto as_global(V *p) {
    return (V __attribute__((address_space(1))) *)p;
}
// one element (the unaligned and ragged paths)
template <typename T>
__device__ __forceinline__ T ld_elem(const T *p, size_t i) {
    return as_global(p)[i];
}
template <typename T>
__device__ __forceinline__ void st_elem(T *p, size_t i, T v) {
    as_global(p)[i] = v;
}
template <class F>
__device__ __forceinline__ R16<F> ld_elem(const R16<F> *p, size_t i) {
    return R16<F>::from_bits(as_global(reinterpret_cast<const uint16_t *>(p))[i]);
}
template <class F>
__device__ __forceinline__ void st_elem(R16<F> *p, size_t i, R16<F> v) {
    as_global(reinterpret_cast<uint16_t *>(p))[i] = v.bits;
}
template <bool NT, typename V>
__device__ __forceinline__ V ld(const V *p) {
    if constexpr (NT) return __builtin_nontemporal_load(as_global(p));
    return *as_global(p);
}
template <bool NT, typename V>
__device__ __forceinline__ void st(V *p, V v) {
    if constexpr (NT)
        __builtin_nontemporal_store(v, as_global(p));
    else
        *as_global(p) = v;
}

// Waits until every memory operation this wave has issued is complete; the compiler may not move
// loads or stores across it.
__device__ __forceinline__ void wait_for_memory() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ float toa_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double toa_sqrt(double x) { return sqrt(x); }
// a 16-bit value picks the float overload; the root is NOT rounded back
template <class F>
__device__ __forceinline__ float toa_sqrt(R16<F> x) { return sqrtf((float)x); }

// as for one 16-bit value: the root is taken in float and NOT rounded back
template <class F>
__device__ __forceinline__ Float2 toa_sqrt(Pair16<F> x) {
    return {sqrtf(x.low()), sqrtf(x.high())};
}

// The step direction mu_hat / (sqrt(nu_hat + eps_root) + eps) as the reference writes it
// (adam_op_impl_cpu.cpp:58-60, 177-179).
template <typename T>
__device__ __forceinline__ T adam_direction(T mh, T vh, T eps_root, T eps) {
    return mh / (toa_sqrt(vh + eps_root) + eps);
}

// bfloat16: the root, the sum with eps and the quotient run in float and only the quotient is
// rounded to 8 significant bits, so the correctly rounded float root and quotient (ten and
// twelve instructions each) are needed only when the quotient lands next to a rounding boundary
// of the 16-bit result.  The quick route takes the hardware's 1-ulp root and reciprocal:
//     s' = sqrt~(x), d' = s' + eps, q' = mu_hat * rcp~(d')
// q' is within 9 float ulps of the exact chain's quotient (1 + 0.5 ulp from the root carried
// through the sum, one rounding of each sum, 1 ulp of the reciprocal, the rounding of each
// product and quotient: 4.5 * 2^-23 relative).  If q' is further than 16 float ulps from the
// midpoint between two bfloat16 values, both round to the same bfloat16 and `ok` is set.
// Otherwise -- about one element in two thousand -- or when an operand is outside the range
// where the 1-ulp claims hold (denormal, zero divisor, infinity, NaN, negative; a negative eps,
// with which root + eps can cancel), the caller runs the exact chain for that element.  Checked against the exact chain for every
// (mu_hat, nu_hat + eps_root) pair of bit patterns.
template <typename T>
struct HasQuickDirection {
    static constexpr bool value = false;
};
template <>
struct HasQuickDirection<bfloat_t> {
    static constexpr bool value = true;
};
template <>
struct HasQuickDirection<half_t> {
    static constexpr bool value = true;
};

__device__ __forceinline__ bfloat_t adam_direction_quick(bfloat_t mh, bfloat_t vh,
                                                         bfloat_t eps_root, bfloat_t eps,
                                                         bool &ok) {
    const bfloat_t x16 = vh + eps_root;
    const float x = (float)x16, m = (float)mh, e = (float)eps;
    const float d = __builtin_amdgcn_sqrtf(x) + e;
    const float q = m * __builtin_amdgcn_rcpf(d);
    const uint32_t low = __builtin_bit_cast(uint32_t, q) & 0xffffu;
    const float aq = __builtin_fabsf(q);
    ok = (x == 0.0f || x >= 1.17549435e-38f) &&          // normal or zero radicand
         e >= 0.0f &&  // no cancellation in root + eps (a negative or NaN eps takes the exact chain)
         d >= 5.42101086e-20f && d <= 1.84467441e19f &&  // 2^-64 .. 2^64
         ((aq >= 7.88860905e-31f && aq <= 1.26765060e30f) || m == 0.0f) &&  // 2^-100 .. 2^100
         (low - 0x7ff0u > 0x20u);  // not within 16 ulps of the midpoint 0x8000
    return bfloat_t(q);
}

// float16 likewise: 11 significant bits, so the midpoints lie 0x2000 float ulps apart (the
// quick route settles fewer elements), and the result must be a normal float16.
__device__ __forceinline__ half_t adam_direction_quick(half_t mh, half_t vh, half_t eps_root,
                                                       half_t eps, bool &ok) {
    const half_t x16 = vh + eps_root;
    const float x = (float)x16, m = (float)mh, e = (float)eps;
    const float d = __builtin_amdgcn_sqrtf(x) + e;
    const float q = m * __builtin_amdgcn_rcpf(d);
    const uint32_t low = __builtin_bit_cast(uint32_t, q) & 0x1fffu;
    const float aq = __builtin_fabsf(q);
    ok = x >= 0.0f && e >= 0.0f && d >= 5.42101086e-20f && d <= 1.84467441e19f &&
         ((aq >= 6.10351562e-05f && aq <= 32768.0f) || m == 0.0f) &&  // 2^-14 .. 2^15
         (low - 0x0ff0u > 0x20u);  // not within 16 ulps of the midpoint 0x1000
    return half_t(q);
}

// The quick route for two values at once; returns the halves that must repeat through the exact
// chain (bit 0: low, bit 1: high).  Same claims as above, with the conditions that do not depend
// on the element checked once: with 2^-64 <= eps <= 2^63 and a radicand that is zero or a positive
// normal number (or eps = 0 and a positive normal radicand), root + eps lies in [2^-64, 2^65] --
// the reciprocal's good range -- whatever the element, so only the radicand's class, the quotient's range and its distance from a rounding
// midpoint remain per element.  Written without short-circuit operators: the compiler then emits
// straight-line compares instead of a branch per element.
template <class F>
struct QuickLimits;
template <>
struct QuickLimits<BFloatFormat> {  // 8 significant bits; any normal float result will do
    static constexpr uint32_t kLowMask = 0xffffu, kMid = 0x8000u;
    static constexpr uint32_t kMinBits = 0x0d800000u, kMaxBits = 0x71800000u;  // 2^-100 .. 2^100
};
template <>
struct QuickLimits<HalfFormat> {  // 11 significant bits; the result must be a normal float16
    static constexpr uint32_t kLowMask = 0x1fffu, kMid = 0x1000u;
    static constexpr uint32_t kMinBits = 0x38800000u, kMaxBits = 0x47000000u;  // 2^-14 .. 2^15
};

template <class F>
__device__ __forceinline__ Pair16<F> adam_direction_quick(Pair16<F> mh, Pair16<F> vh,
                                                          Pair16<F> eps_root, Pair16<F> eps,
                                                          uint32_t &bad) {
    using L = QuickLimits<F>;
    const Pair16<F> x = vh + eps_root;
    const float e = eps.low();  // both halves hold the same hyper-parameter
    // eps = 0 is served too: the radicand must then be positive (a zero one would divide by zero)
    const bool eps_fits = ((e >= 5.42101086e-20f) & (e <= 9.22337204e18f)) | (e == 0.0f);
    const int radicand_classes = e == 0.0f ? 0x100 : 0x160;
    auto one = [&](float xx, float m, float &q) -> bool {
        const float d = __builtin_amdgcn_sqrtf(xx) + e;
        q = m * __builtin_amdgcn_rcpf(d);
        const uint32_t qb = __builtin_bit_cast(uint32_t, q);
        const uint32_t aq = qb & 0x7fffffffu;
        // zero or a positive normal radicand (class bits: +normal 0x100, +0 0x040, -0 0x020)
        const bool radicand = __builtin_amdgcn_classf(xx, radicand_classes);
        const bool range = (aq - L::kMinBits <= L::kMaxBits - L::kMinBits) | (aq == 0u);
        // not within 16 float ulps of the midpoint between two 16-bit values
        const bool clear = ((qb & L::kLowMask) - (L::kMid - 0x10u)) > 0x20u;
        return radicand & range & clear;
    };
    float q_lo, q_hi;
    const bool ok_lo = one(x.low(), mh.low(), q_lo) & eps_fits;
    const bool ok_hi = one(x.high(), mh.high(), q_hi) & eps_fits;
    bad = (ok_lo ? 0u : 1u) | (ok_hi ? 0u : 2u);
    return Pair16<F>::rounded(q_lo, q_hi);
}

// An op is speculative when it offers `quick(in, out) -> bool` beside the exact operator():
// the whole-tile path runs quick() on every element and repeats only the elements that
// returned false with the exact operator.
template <class Op, class = void>
struct IsSpeculative {
    static constexpr bool value = false;
};
template <class Op>
struct IsSpeculative<Op, decltype((void)Op::kSpeculative)> {
    static constexpr bool value = Op::kSpeculative;
};

// An op is staged when its three outputs come from three steps that need the inputs one after
// the other:  a = first(in0, in1),  b = second(in0, in2),  c = third(a, b)  (third_quick for the
// speculative 16-bit route).  tile_full_staged() stores a and b as soon as they exist.
template <class Op, class = void>
struct IsStaged {
    static constexpr bool value = false;
};
template <class Op>
struct IsStaged<Op, decltype((void)Op::kStaged)> {
    static constexpr bool value = Op::kStaged;
};

// ---------------------------------------------------------------------------
// Step number on the device.  The reference keeps `count` as a 0-dim device tensor
// (/root/reference/torchopt/transform/scale_by_adam.py:401-414) and reads it back on every call;
// the ordinary entry points here take it as a host integer, which a captured graph would freeze.
// An op wrapped in AtStep reads the step number from device memory when its kernel starts and
// takes its bias corrections from a table of rows {c1, c2, p1, q2} that the host filled for
// steps first, first + 1, ... (in double with libm's pow, rounded to the element type: the same
// values the host-count entry points put into kernel arguments).  Steps before `first` use the
// first row, steps beyond the table the last one.
// ---------------------------------------------------------------------------
template <typename T>
struct StepRef {
    const T *rows;         // 4 values per row
    const int64_t *count;  // the step number of this step
    int64_t first;         // step number of row 0
    int64_t last_row;
};

// wave-uniform loads through the constant address space: the scalar unit's
__device__ __forceinline__ float load_uniform(const float *p) {
    return *(const __attribute__((address_space(4))) float *)p;
}
__device__ __forceinline__ double load_uniform(const double *p) {
    return *(const __attribute__((address_space(4))) double *)p;
}
__device__ __forceinline__ uint32_t load_uniform(const uint32_t *p) {
    return *(const __attribute__((address_space(4))) uint32_t *)p;
}
__device__ __forceinline__ int64_t load_uniform(const int64_t *p) {
    return *(const __attribute__((address_space(4))) int64_t *)p;
}
template <class F>
__device__ __forceinline__ R16<F> load_uniform(const R16<F> *p) {
    return R16<F>::from_bits(*(const __attribute__((address_space(4))) uint16_t *)p);
}

template <class Op, typename T>
struct AtStep : Op {
    StepRef<T> step;
    __device__ __forceinline__ void fetch() {
        int64_t r = load_uniform(step.count) - step.first;
        r = r < 0 ? 0 : (r > step.last_row ? step.last_row : r);
        const T *row = step.rows + 4 * r;
        this->set_bias(load_uniform(row), load_uniform(row + 1), load_uniform(row + 2),
                       load_uniform(row + 3));
    }
};
template <class Op>
struct FetchesStep {
    static constexpr bool value = false;
};
template <class Op, typename T>
struct FetchesStep<AtStep<Op, T>> {
    static constexpr bool value = true;
};
// The op a kernel computes with: the launch's op, with the bias corrections of the current step
// filled in where the step number lives on the device.
template <class Op>
__device__ __forceinline__ Op live_op(const Op &op) {
    Op live = op;
    if constexpr (FetchesStep<Op>::value) live.fetch();
    return live;
}

// Load orders of an op's staged program (1 unless the op says otherwise).
template <class Op, class = void>
struct LoadOrders {
    static constexpr int value = 1;
};
template <class Op>
struct LoadOrders<Op, decltype((void)Op::kLoadOrders)> {
    static constexpr int value = Op::kLoadOrders;
};

// What a staged op sees of its tile: one 128-bit vector per lane of every array.
template <typename T, class Op, bool NT>
struct StagedIO {
    using V = typename Vec<T>::type;
    T *const *p;  // the tensor's pointer slots
    size_t v0;    // this lane's vector index
    __device__ __forceinline__ V load(int slot) const {
        return ld<NT>(reinterpret_cast<const V *>(p[slot]) + v0);
    }
    __device__ __forceinline__ void store(int slot, V x) const {
        st<NT>(reinterpret_cast<V *>(p[slot]) + v0, x);
    }
    // every memory operation issued so far is complete; nothing moves across
    __device__ __forceinline__ void wait() const { wait_for_memory(); }
};

// r[e] = f(a[e], b[e]) over the elements of two vectors
template <typename T, class F>
__device__ __forceinline__ typename Vec<T>::type vmap(const typename Vec<T>::type &a,
                                                      const typename Vec<T>::type &b, F f) {
    typename Vec<T>::type r;
#pragma unroll
    for (int e = 0; e < Vec<T>::N; ++e) Vec<T>::set(r, e, f(Vec<T>::get(a, e), Vec<T>::get(b, e)));
    return r;
}

// Residency level by element type, measured per op: float32, float64, float16, bfloat16.  (The
// 16-bit types spend more ALU time per byte on re-rounding, bfloat16 the most.)
template <typename T>
constexpr int waves_by_type(int f32, int f64, int half, int bfloat) {
    return sizeof(T) == 4 ? f32 : sizeof(T) == 8 ? f64 : (__is_same(T, bfloat_t) ? bfloat : half);
}
// The multi-tensor kernel's levels were measured on their own: float32 / float64, float16, bfloat16.
template <typename T>
constexpr int waves_by_type(int wide, int half, int bfloat) {
    return waves_by_type<T>(wide, wide, half, bfloat);
}

// ---------------------------------------------------------------------------
// Element-wise ops.  Pointer slots: inputs first, then outputs; an in-place op
// writes output j back to input slot out_slot(j).  kWavesPerCU / kWavesPerCUMulti are the measured
// best number of resident single-wave workgroups per compute unit.
// ---------------------------------------------------------------------------

// The three steps of one Adam update as the reference writes them (adam_op_impl_cpu.cpp:47-61):
// the two moments, then the step direction from the bias-corrected moments.  Shared by the
// in-place step and the one-pass differentiable forward.
// (Ops are aligned to 8 bytes whatever their element type: a kernel argument of 2-byte alignment --
// an op over a 16-bit type -- would be fetched with a VECTOR load, whose latency the list kernels
// pay in full before they can even look up their tensor; aligned, it comes through the scalar
// unit like every other argument.)
template <typename T>
struct alignas(8) AdamSteps {
    T b1, b2, c1, c2, eps, eps_root;
    __device__ __forceinline__ void set_bias(T c1_, T c2_, T, T) {
        c1 = c1_;
        c2 = c2_;
    }
    // U is T, or for the 16-bit types the pair type that computes two elements side by side
    template <class U>
    __device__ __forceinline__ U first(U g, U m) const {
        return U(b1) * m + (1 - U(b1)) * g;
    }
    template <class U>
    __device__ __forceinline__ U second(U g, U v) const {
        return U(b2) * v + (1 - U(b2)) * g * g;
    }
    template <class U>
    __device__ __forceinline__ U third(U m1, U v1) const {
        const U mh = m1 * U(c1);
        const U vh = v1 * U(c2);
        return adam_direction(mh, vh, U(eps_root), U(eps));
    }
    // two elements through all three steps, the third by the quick route; returns the halves
    // that must repeat through the exact chain (bit 0, bit 1)
    template <class P>
    __device__ __forceinline__ uint32_t quick_pair(const P (&in)[3], P (&out)[3]) const {
        out[0] = first<P>(in[0], in[1]);
        out[1] = second<P>(in[0], in[2]);
        return third_quick_pair<P>(out[0], out[1], out[2]);
    }
    template <class P>
    __device__ __forceinline__ uint32_t third_quick_pair(P m1, P v1, P &out) const {
        const P mh = m1 * P(c1);
        const P vh = v1 * P(c2);
        uint32_t bad;
        out = adam_direction_quick(mh, vh, P(eps_root), P(eps), bad);
        return bad;
    }
    __device__ __forceinline__ bool third_quick(T m1, T v1, T &out) const {
        const T mh = m1 * c1;
        const T vh = v1 * c2;
        bool ok = true;
        if constexpr (HasQuickDirection<T>::value)
            out = adam_direction_quick(mh, vh, eps_root, eps, ok);
        else
            out = adam_direction(mh, vh, eps_root, eps);
        return ok;
    }
    // load in0 | load in1 | store out0, load in2 | store out1, store out2 (ORDER 0; see below)
    template <class Op, int ORDER = 0, class IO>
    __device__ __forceinline__ void staged_steps(const IO &io) const {
        using V = typename Vec<T>::type;
        constexpr int VN = Vec<T>::N;
        if constexpr (sizeof(T) == 2) {
            // the 16-bit types: two elements per step (see Pair16: bfloat16 rounds a pair with
            // one instruction, float16 computes in packed half arithmetic), the quick route for
            // both elements
            using P = typename PairOf<T>::type;
            typedef uint32_t Words __attribute__((ext_vector_type(4)));
            const Words g = __builtin_bit_cast(Words, io.load(0));
            io.wait();
            const Words m = __builtin_bit_cast(Words, io.load(1));
            io.wait();
            P gp[4], ap[4], bp[4];
            Words a, b, c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                gp[e] = P::from_bits(g[e]);
                ap[e] = first<P>(gp[e], P::from_bits(m[e]));
                a[e] = ap[e].bits();
            }
            io.store(Op::out_slot(0), __builtin_bit_cast(V, a));
            const Words v = __builtin_bit_cast(Words, io.load(2));
            io.wait();
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                bp[e] = second<P>(gp[e], P::from_bits(v[e]));
                b[e] = bp[e].bits();
            }
            io.store(Op::out_slot(1), __builtin_bit_cast(V, b));
            uint32_t redo = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                P r;
                redo |= third_quick_pair<P>(ap[e], bp[e], r) << (2 * e);
                c[e] = r.bits();
            }
            V res = __builtin_bit_cast(V, c);
            if (redo != 0) {  // rare: an element the quick route could not settle
                const V av = __builtin_bit_cast(V, a), bv = __builtin_bit_cast(V, b);
#pragma unroll
                for (int e = 0; e < VN; ++e)
                    if (redo & (1u << e))
                        Vec<T>::set(res, e, third<T>(Vec<T>::get(av, e), Vec<T>::get(bv, e)));
            }
            io.store(Op::out_slot(2), res);
        } else {
            // ORDER picks which moment is handled first and whether it is loaded before the
            // gradient: 0 = g, mu, nu; 1 = g, nu, mu; 2 = mu, g, nu; 3 = nu, g, mu.  The results
            // do not depend on it.
            constexpr bool nu_first = ORDER == 1 || ORDER == 3;
            constexpr bool moment_before_gradient = ORDER >= 2;
            constexpr int in_a = nu_first ? 2 : 1, in_b = nu_first ? 1 : 2;
            constexpr int out_a = nu_first ? 1 : 0, out_b = nu_first ? 0 : 1;
            auto moment = [&](bool second_moment, const V &gg, const V &x) {
                return second_moment ? vmap<T>(gg, x, [&](T p, T q) { return second<T>(p, q); })
                                     : vmap<T>(gg, x, [&](T p, T q) { return first<T>(p, q); });
            };
            V g, xa;
            if constexpr (moment_before_gradient) {
                xa = io.load(in_a);
                io.wait();
                g = io.load(0);
                io.wait();
            } else {
                g = io.load(0);
                io.wait();
                xa = io.load(in_a);
                io.wait();
            }
            const V ra = moment(nu_first, g, xa);
            io.store(Op::out_slot(out_a), ra);
            const V xb = io.load(in_b);
            io.wait();
            const V rb = moment(!nu_first, g, xb);
            io.store(Op::out_slot(out_b), rb);
            const V &a = nu_first ? rb : ra;  // the new first moment
            const V &b = nu_first ? ra : rb;  // the new second moment
            V c;
            if constexpr (HasQuickDirection<T>::value) {
                uint32_t redo = 0;
#pragma unroll
                for (int e = 0; e < VN; ++e) {
                    T r;
                    if (!third_quick(Vec<T>::get(a, e), Vec<T>::get(b, e), r)) redo |= 1u << e;
                    Vec<T>::set(c, e, r);
                }
                if (redo != 0) {  // rare: an element the quick route could not settle
#pragma unroll
                    for (int e = 0; e < VN; ++e)
                        if (redo & (1u << e))
                            Vec<T>::set(c, e, third<T>(Vec<T>::get(a, e), Vec<T>::get(b, e)));
                }
            } else {
                c = vmap<T>(a, b, [&](T x, T y) { return third<T>(x, y); });
            }
            io.store(Op::out_slot(2), c);
        }
    }
    template <bool QUICK>
    __device__ __forceinline__ bool run(const T (&in)[3], T (&out)[3]) const {
        out[0] = first<T>(in[0], in[1]);
        out[1] = second<T>(in[0], in[2]);
        if constexpr (QUICK) return third_quick(out[0], out[1], out[2]);
        out[2] = third<T>(out[0], out[1]);
        return true;
    }
    __device__ __forceinline__ void operator()(const T (&in)[3], T (&out)[3]) const {
        run<false>(in, out);
    }
    __device__ __forceinline__ bool quick(const T (&in)[3], T (&out)[3]) const {
        return run<true>(in, out);
    }
};

// adam_op_impl_cpu.cpp:47-61.  Slots: 0 updates, 1 mu, 2 nu.
template <typename T>
struct ForwardInplace : AdamSteps<T> {
    static constexpr int NIN = 3, NOUT = 3, NPTR = 3;
    // read-modify-write: a tight window wins
    static constexpr int kWavesPerCU = waves_by_type<T>(12, 10, 16, 14);
    static constexpr int kWavesPerCUMulti = waves_by_type<T>(16, 25, 25);
    static constexpr bool kStaged = true;
    static constexpr int kWavesPerCUStaged = waves_by_type<T>(18, 18, 21, 21);
    // A float32 / float64 list gains nothing from the staged schedule (6.5-6.6 TB/s either way
    // on the GPT-2-medium list) unless its arrays collide in DRAM, so such lists are staged only
    // then; the 16-bit lists gain 1-2 % from it at 25 waves per CU (measured after 100 launches of
    // the same kind: the first 40-50 launches of a 16-bit kernel run up to 6 % slower).
    static constexpr bool kStagedLists = sizeof(T) == 2;
    static constexpr int kWavesPerCUStagedLists = waves_by_type<T>(18, 18, 25, 25);
    // outputs are produced as (mu', nu', updates') and stored in that order
    __device__ static constexpr int out_slot(int j) { return j == 0 ? 1 : (j == 1 ? 2 : 0); }
    static constexpr bool kSpeculative = HasQuickDirection<T>::value;
    static constexpr bool kPairs = true;
    // The staged program exists in four load orders (the 16-bit types, which compute in pairs, in
    // one): which order streams fastest depends on where the three arrays lie, see staged_steps.
    static constexpr int kLoadOrders = sizeof(T) == 2 ? 1 : 4;
    template <class IO>
    __device__ __forceinline__ void staged(const IO &io) const {
        this->template staged_steps<ForwardInplace, 0>(io);
    }
    template <int ORDER, class IO>
    __device__ __forceinline__ void staged_in_order(const IO &io) const {
        this->template staged_steps<ForwardInplace, ORDER>(io);
    }
};

// adam_op_impl_cpu.cpp:103-108.  Slots: 0 updates, 1 mu, 2 mu_out.
template <typename T>
struct alignas(8) ForwardMu {
    static constexpr int NIN = 2, NOUT = 1, NPTR = 3;
    static constexpr int kWavesPerCU = 25;
    static constexpr int kWavesPerCUMulti = 32;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T b1;
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        out[0] = b1 * in[1] + (1 - b1) * in[0];
    }
};

// adam_op_impl_cpu.cpp:137-143.  Slots: 0 updates, 1 nu, 2 nu_out.
template <typename T>
struct alignas(8) ForwardNu {
    static constexpr int NIN = 2, NOUT = 1, NPTR = 3;
    static constexpr int kWavesPerCU = waves_by_type<T>(21, 21, 32, 32);
    static constexpr int kWavesPerCUMulti = 32;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T b2;
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        const T g = in[0];
        out[0] = b2 * in[1] + (1 - b2) * g * g;
    }
};

// adam_op_impl_cpu.cpp:175-181.  Slots: 0 new_mu, 1 new_nu, 2 updates_out.
template <typename T>
struct alignas(8) ForwardUpdates {
    static constexpr int NIN = 2, NOUT = 1, NPTR = 3;
    // root and quotient: the 16-bit types need every wave to hide the ALU time
    static constexpr int kWavesPerCU = waves_by_type<T>(21, 18, 32, 32);
    static constexpr int kWavesPerCUMulti = 32;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    static constexpr bool kSpeculative = HasQuickDirection<T>::value;
    static constexpr bool kPairs = true;
    T c1, c2, eps, eps_root;
    template <class P>
    __device__ __forceinline__ uint32_t quick_pair(const P (&in)[NIN], P (&out)[NOUT]) const {
        const P mh = in[0] * P(c1);
        const P vh = in[1] * P(c2);
        uint32_t bad;
        out[0] = adam_direction_quick(mh, vh, P(eps_root), P(eps), bad);
        return bad;
    }
    template <bool QUICK>
    __device__ __forceinline__ bool run(const T (&in)[NIN], T (&out)[NOUT]) const {
        const T mh = in[0] * c1;
        const T vh = in[1] * c2;
        bool ok = true;
        if constexpr (QUICK)
            out[0] = adam_direction_quick(mh, vh, eps_root, eps, ok);
        else
            out[0] = adam_direction(mh, vh, eps_root, eps);
        return ok;
    }
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        run<false>(in, out);
    }
    __device__ __forceinline__ bool quick(const T (&in)[NIN], T (&out)[NOUT]) const {
        return run<true>(in, out);
    }
};

// adam_op_impl_cpu.cpp:220-226.  Slots: 0 dmu, 1 dupdates_out, 2 dmu_out.
template <typename T>
struct alignas(8) BackwardMu {
    static constexpr int NIN = 1, NOUT = 2, NPTR = 3;
    static constexpr int kWavesPerCU = 18;
    static constexpr int kWavesPerCUMulti = 25;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T b1;
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        out[0] = (1 - b1) * in[0];
        out[1] = b1 * in[0];
    }
};

// adam_op_impl_cpu.cpp:257-264.  Slots: 0 dnu, 1 updates, 2 dupdates_out, 3 dnu_out.
template <typename T>
struct alignas(8) BackwardNu {
    static constexpr int NIN = 2, NOUT = 2, NPTR = 4;
    static constexpr int kWavesPerCU = 16;
    static constexpr int kWavesPerCUMulti = 25;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T b2;
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        out[0] = 2 * (1 - b2) * in[1] * in[0];
        out[1] = b2 * in[0];
    }
};

// adam_op_impl_cpu.cpp:298-316.  Slots: 0 dupdates, 1 updates, 2 new_mu,
// 3 dnew_mu_out, 4 dnew_nu_out.  p1 = 1 - b1^count, q2 = 1/(1 - b2^count + eps_root).
template <typename T>
struct alignas(8) BackwardUpdates {
    static constexpr int NIN = 3, NOUT = 2, NPTR = 5;
    static constexpr int kWavesPerCU = waves_by_type<T>(18, 12, 16, 16);
    static constexpr int kWavesPerCUMulti = 25;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T p1, q2;
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        const T d = in[0], u = in[1], m1 = in[2];
        const T r = u / m1;
        const T den = r * p1;
        const T dm = d * r;
        // two products in T, then the double literal 0.5 lifts the rest to double
        const T dn = static_cast<T>(-d * u * den * 0.5 * q2 * den);
        const bool zero = (m1 == 0);  // +0 and -0, not NaN
        out[0] = zero ? T(0) : dm;
        out[1] = zero ? T(0) : dn;
    }
};

// The whole differentiable forward of one step in one pass: what forward_mu, forward_nu and
// forward_updates produce, from one read of updates, mu and nu (24 instead of 36 bytes per
// float32 element, one launch instead of three).  Same expressions as ForwardInplace, written
// to fresh outputs.  Slots: 0 updates, 1 mu, 2 nu, 3 new_mu, 4 new_nu, 5 new_updates.
template <typename T>
struct ForwardAll : AdamSteps<T> {
    static constexpr int NIN = 3, NOUT = 3, NPTR = 6;
    static constexpr int kWavesPerCU = waves_by_type<T>(11, 10, 16, 14);  // six streams per wave: few waves fill the queues
    static constexpr int kWavesPerCUMulti = waves_by_type<T>(18, 21, 32);
    // measured: float64 6.75 against 6.55 TB/s, float16 6.69 against 6.46; float32 loses
    // (6.45 against 6.62) and bfloat16 is bound by its arithmetic
    static constexpr bool kStaged = __is_same(T, double) || __is_same(T, half_t);
    static constexpr int kWavesPerCUStaged = waves_by_type<T>(18, 18, 21, 32);
    static constexpr bool kStagedLists = false;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    static constexpr bool kSpeculative = HasQuickDirection<T>::value;
    static constexpr bool kPairs = true;
    template <class IO>
    __device__ __forceinline__ void staged(const IO &io) const {
        this->template staged_steps<ForwardAll>(io);
    }
};

// The whole backward of that step in one pass: backward_updates, the two sums autograd would
// form (gradient arriving at new_mu / new_nu from elsewhere plus the one from the update), then
// backward_mu and backward_nu and the sum of their two contributions to d(updates) -- each
// still rounded on its own, so the result equals the three separate passes plus autograd's
// additions bit for bit.  HAS_DM / HAS_DV say whether an outside gradient for new_mu / new_nu
// exists; without one the sum is skipped, exactly as autograd skips it.
// Slots: 0 d(new_updates), 1 new_updates, 2 new_mu, 3 updates, [d(new_mu)], [d(new_nu)],
// then outputs d(updates), d(mu), d(nu).
template <typename T, bool HAS_DM, bool HAS_DV>
struct alignas(8) BackwardAll {
    static constexpr int NIN = 4 + (HAS_DM ? 1 : 0) + (HAS_DV ? 1 : 0), NOUT = 3,
                         NPTR = NIN + NOUT;
    static constexpr int kWavesPerCU = waves_by_type<T>(10, 10, 12, 12);  // seven to nine streams per wave
    static constexpr int kWavesPerCUMulti = waves_by_type<T>(14, 16, 16);
    // staged: float32 / float64 only (the 16-bit types are bound by their arithmetic here)
    static constexpr bool kStaged = sizeof(T) >= 4;
    // the more streams a wave carries, the fewer waves fill the queues: nine streams 12, seven 16
    static constexpr int kWavesPerCUStaged = HAS_DM && HAS_DV ? 12 : (HAS_DM || HAS_DV ? 14 : 16);
    static constexpr bool kStagedLists = false;
    __device__ static constexpr int out_slot(int j) { return NIN + j; }
    T b1, b2, p1, q2;
    __device__ __forceinline__ void set_bias(T, T, T p1_, T q2_) {
        p1 = p1_;
        q2 = q2_;
    }
    // d(new_mu) and d(new_nu) arriving from the update: backward_updates
    __device__ __forceinline__ void from_update(T d, T u, T m1, T &tot_m, T &tot_v) const {
        const T r = u / m1;
        const T den = r * p1;
        const bool zero = (m1 == 0);
        tot_m = zero ? T(0) : T(d * r);
        tot_v = zero ? T(0) : static_cast<T>(-d * u * den * 0.5 * q2 * den);
    }
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        const T g = in[3];
        T tot_m, tot_v;
        from_update(in[0], in[1], in[2], tot_m, tot_v);
        if constexpr (HAS_DM) tot_m = in[4] + tot_m;
        if constexpr (HAS_DV) tot_v = in[HAS_DM ? 5 : 4] + tot_v;
        const T du_from_mu = (1 - b1) * tot_m;
        const T du_from_nu = 2 * (1 - b2) * g * tot_v;
        out[0] = du_from_mu + du_from_nu;
        out[1] = b1 * tot_m;
        out[2] = b2 * tot_v;
    }
    // load d(new_updates), new_updates | load new_mu [, d(new_mu)] | store d(mu),
    // load updates [, d(new_nu)] | store d(nu), store d(updates)
    template <class IO>
    __device__ __forceinline__ void staged(const IO &io) const {
        using V = typename Vec<T>::type;
        constexpr int VN = Vec<T>::N;
        const V d = io.load(0);
        const V u = io.load(1);
        io.wait();
        const V m1 = io.load(2);
        V dm, dv;
        if constexpr (HAS_DM) dm = io.load(4);
        io.wait();
        T tot_m[VN], tot_v[VN];
        V dmu;
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            from_update(Vec<T>::get(d, e), Vec<T>::get(u, e), Vec<T>::get(m1, e), tot_m[e],
                        tot_v[e]);
            if constexpr (HAS_DM) tot_m[e] = Vec<T>::get(dm, e) + tot_m[e];
            Vec<T>::set(dmu, e, b1 * tot_m[e]);
        }
        io.store(out_slot(1), dmu);
        const V g = io.load(3);
        if constexpr (HAS_DV) dv = io.load(HAS_DM ? 5 : 4);
        io.wait();
        V dnu, du;
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            if constexpr (HAS_DV) tot_v[e] = Vec<T>::get(dv, e) + tot_v[e];
            Vec<T>::set(dnu, e, b2 * tot_v[e]);
            const T du_from_mu = (1 - b1) * tot_m[e];
            const T du_from_nu = 2 * (1 - b2) * Vec<T>::get(g, e) * tot_v[e];
            Vec<T>::set(du, e, du_from_mu + du_from_nu);
        }
        io.store(out_slot(2), dnu);
        io.store(out_slot(0), du);
    }
};

// The classic optimizer step in one pass: the in-place Adam step together with what
// the reference chains do around it --
//   [maximize]        g = -g                       alias/utils.py:148
//   [L2 decay, adam]  g = g + wd * p               alias/utils.py:113-122
//   Adam forward_                                  adam_op_impl_cpu.cpp:32-91
//   [decay, adamw]    u = u + wd * p               transform/add_decayed_weights.py:232-239
//   u = u * (-lr)                                  transform/scale.py:93-98
//   p = p + u                                      update.py:71-74
// (paths under /root/reference/torchopt) -- each still rounded as the separate
// passes round it, so the result equals them bit for bit while streaming 28 (or
// 32) bytes per float32 element instead of 44 and more.  The two "+ wd * p" are
// single-rounding fused multiply-adds because that is what Tensor.add_(p,
// alpha=wd) computes, on CPU and GPU alike; everything else is one rounding per
// operation.
// Slots: 0 updates (gradients), 1 mu, 2 nu, 3 params.
enum : int { kNoDecay = 0, kDecayIntoGradient = 1, kDecayIntoUpdate = 2 };

__device__ __forceinline__ float toa_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double toa_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
// 16-bit tensors: PyTorch evaluates Tensor.add_(p, alpha=wd) and Tensor.mul_(-lr) in float -- the
// Python scalar goes double -> float and is NOT rounded to 16 bits, the tensor operands widen, one
// float operation (a fused multiply-add for add_), one rounding back to 16 bits.  The float result
// of these overloads is rounded when it is assigned to the 16-bit type.
template <class F>
__device__ __forceinline__ float toa_fma(float a, R16<F> b, R16<F> c) {
    return rounded_to_float(__builtin_fmaf(a, (float)b, (float)c));
}
// The type the step's two scalars (-lr and the weight decay) are held in: the element type for
// float32 / float64, float for the 16-bit types.
template <typename T>
struct StepScalarOf {
    using type = T;
};
template <class F>
struct StepScalarOf<R16<F>> {
    using type = float;
};
template <typename T>
using StepScalar = typename StepScalarOf<T>::type;

template <typename T, bool WRITE_UPDATES>
struct alignas(8) FusedStep {
    static constexpr int NIN = 4, NOUT = WRITE_UPDATES ? 4 : 3, NPTR = 4;
    static constexpr int kWavesPerCU = waves_by_type<T>(12, 10, 12, 12);
    static constexpr int kWavesPerCUMulti = 16;
    // staged: 6.77 against 6.66 TB/s on one tensor, 6.61 against 6.41 on the GPT-2-medium list
    static constexpr bool kStaged = true;
    static constexpr int kWavesPerCUStaged = 21;
    static constexpr bool kStagedLists = true;
    // outputs: mu', nu', params', then the scaled update
    __device__ static constexpr int out_slot(int j) { return j == 3 ? 0 : j + 1; }
    T b1, b2, c1, c2, eps, eps_root;
    StepScalar<T> neg_lr, wd;
    int decay;
    bool maximize;
    __device__ __forceinline__ void set_bias(T c1_, T c2_, T, T) {
        c1 = c1_;
        c2 = c2_;
    }
    // the gradient the moments see
    __device__ __forceinline__ T gradient(T g, T p) const {
        g = maximize ? -g : g;
        if (decay == kDecayIntoGradient) g = toa_fma(wd, p, g);
        return g;
    }
    __device__ __forceinline__ T first(T g, T m) const { return b1 * m + (1 - b1) * g; }
    __device__ __forceinline__ T second(T g, T v) const { return b2 * v + (1 - b2) * g * g; }
    __device__ __forceinline__ T direction(T m1, T v1) const {
        const T mh = m1 * c1;
        const T vh = v1 * c2;
        if constexpr (HasQuickDirection<T>::value) {
            // the checked shortcut of the 16-bit types; an element it cannot settle takes the
            // exact chain
            bool ok;
            const T quick = adam_direction_quick(mh, vh, eps_root, eps, ok);
            if (ok) return quick;
        }
        return adam_direction(mh, vh, eps_root, eps);
    }
    // the scaled update from the direction
    __device__ __forceinline__ T scaled(T u1, T p) const {
        if (decay == kDecayIntoUpdate) u1 = toa_fma(wd, p, u1);
        return u1 * neg_lr;
    }
    __device__ __forceinline__ void operator()(const T (&in)[NIN], T (&out)[NOUT]) const {
        const T p = in[3];
        const T g = gradient(in[0], p);
        const T m1 = first(g, in[1]);
        const T v1 = second(g, in[2]);
        const T step = scaled(direction(m1, v1), p);
        out[0] = m1;
        out[1] = v1;
        out[2] = p + step;
        if constexpr (WRITE_UPDATES) out[3] = step;
    }
    // load g [and p, when the gradient needs it] | load mu | store mu', load nu |
    // store nu', load p | store p' [and the scaled update]
    template <class IO>
    __device__ __forceinline__ void staged(const IO &io) const {
        using V = typename Vec<T>::type;
        if constexpr (sizeof(T) == 2) {
            // The 16-bit types (which take no weight decay): two elements per step, as the
            // in-place step computes them (Pair16), the quick route for the direction.
            // load g | load mu | store mu', load nu | store nu', load p | store p' [, store u']
            using P = typename PairOf<T>::type;
            typedef uint32_t Words __attribute__((ext_vector_type(4)));
            constexpr int VN = Vec<T>::N;
            const AdamSteps<T> adam{b1, b2, c1, c2, eps, eps_root};
            Words g = __builtin_bit_cast(Words, io.load(0));
            io.wait();
            if (maximize) g ^= 0x80008000u;  // -g: the sign bit of both halves
            const Words m = __builtin_bit_cast(Words, io.load(1));
            io.wait();
            P gp[4], ap[4], bp[4];
            Words a, b, c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                gp[e] = P::from_bits(g[e]);
                ap[e] = adam.template first<P>(gp[e], P::from_bits(m[e]));
                a[e] = ap[e].bits();
            }
            io.store(1, __builtin_bit_cast(V, a));
            const Words v = __builtin_bit_cast(Words, io.load(2));
            io.wait();
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                bp[e] = adam.template second<P>(gp[e], P::from_bits(v[e]));
                b[e] = bp[e].bits();
            }
            io.store(2, __builtin_bit_cast(V, b));
            const Words p = __builtin_bit_cast(Words, io.load(3));
            uint32_t redo = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                P r;
                redo |= adam.template third_quick_pair<P>(ap[e], bp[e], r) << (2 * e);
                c[e] = r.bits();
            }
            V dir = __builtin_bit_cast(V, c);
            if (redo != 0) {  // rare: an element the quick route could not settle
                const V av = __builtin_bit_cast(V, a), bv = __builtin_bit_cast(V, b);
#pragma unroll
                for (int e = 0; e < VN; ++e)
                    if (redo & (1u << e))
                        Vec<T>::set(dir, e,
                                    adam.template third<T>(Vec<T>::get(av, e), Vec<T>::get(bv, e)));
            }
            io.wait();
            const Words d = __builtin_bit_cast(Words, dir);
            Words p1, step;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // the update times float(-lr), rounded once; then params plus that, rounded once
                const P st(P::from_bits(d[e]) * Float2{neg_lr, neg_lr});
                step[e] = st.bits();
                p1[e] = (P::from_bits(p[e]) + st).bits();
            }
            io.store(3, __builtin_bit_cast(V, p1));
            if constexpr (WRITE_UPDATES) io.store(0, __builtin_bit_cast(V, step));
            return;
        }
        const bool early_p = decay == kDecayIntoGradient;
        V g = io.load(0);
        V p;
        if (early_p) p = io.load(3);
        io.wait();
        if (early_p || maximize) {
            if (!early_p) p = g;  // any value: gradient() ignores it without that decay
            g = vmap<T>(g, p, [&](T x, T y) { return gradient(x, y); });
        }
        const V m = io.load(1);
        io.wait();
        const V m1 = vmap<T>(g, m, [&](T x, T y) { return first(x, y); });
        io.store(1, m1);
        const V v = io.load(2);
        io.wait();
        const V v1 = vmap<T>(g, v, [&](T x, T y) { return second(x, y); });
        io.store(2, v1);
        if (!early_p) p = io.load(3);
        const V u1 = vmap<T>(m1, v1, [&](T x, T y) { return direction(x, y); });
        if (!early_p) io.wait();
        const V step = vmap<T>(u1, p, [&](T x, T y) { return scaled(x, y); });
        const V p1 = vmap<T>(p, step, [&](T x, T y) { return x + y; });
        io.store(3, p1);
        if constexpr (WRITE_UPDATES) io.store(0, step);
    }
};

// The 16-bit instantiations of the ops built on AdamSteps compute whole tiles pair-wise.
template <typename T, class Op, class = void>
struct UsesPairs {
    static constexpr bool value = false;
};
template <class F, class Op>
struct UsesPairs<R16<F>, Op, decltype((void)Op::kPairs)> {
    static constexpr bool value = Op::kPairs;
};

// ---------------------------------------------------------------------------
// Tile processing.  A tile is kBlock * UNROLL vectors (that * Vec<T>::N
// elements) of one tensor; the library instantiates UNROLL = 1.
// ---------------------------------------------------------------------------

template <typename T, int UNROLL>
struct Tile {
    static constexpr int VN = Vec<T>::N;
    static constexpr int VECS = kBlock * UNROLL;
    static constexpr int ELEMS = VECS * VN;
};

template <typename T, class Op>
struct TensorPtrs {
    T *p[Op::NPTR];
};

// All pointers 16-byte aligned, whole tile inside the tensor.
template <typename T, class Op, int UNROLL, bool NT>
__device__ __forceinline__ void tile_full(const Op &op, const TensorPtrs<T, Op> &tp,
                                          size_t vec_base) {
    using V = typename Vec<T>::type;
    constexpr int VN = Vec<T>::N;
    V in[Op::NIN][UNROLL];
    const size_t v0 = vec_base + threadIdx.x;
#pragma unroll
    for (int k = 0; k < UNROLL; ++k)
#pragma unroll
        for (int i = 0; i < Op::NIN; ++i)
            in[i][k] = ld<NT>(reinterpret_cast<const V *>(tp.p[i]) + v0 + (size_t)k * kBlock);

    if constexpr (UsesPairs<T, Op>::value && UNROLL == 1) {
        // a 16-bit op with a pair form: two elements per step, the quick route for both
        using P = typename PairOf<T>::type;
        typedef uint32_t Words __attribute__((ext_vector_type(4)));
        Words w[Op::NIN], o[Op::NOUT];
#pragma unroll
        for (int i = 0; i < Op::NIN; ++i) w[i] = __builtin_bit_cast(Words, in[i][0]);
        uint32_t redo = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            P a[Op::NIN], r[Op::NOUT];
#pragma unroll
            for (int i = 0; i < Op::NIN; ++i) a[i] = P::from_bits(w[i][e]);
            redo |= op.quick_pair(a, r) << (2 * e);
#pragma unroll
            for (int j = 0; j < Op::NOUT; ++j) o[j][e] = r[j].bits();
        }
        V res[Op::NOUT];
#pragma unroll
        for (int j = 0; j < Op::NOUT; ++j) res[j] = __builtin_bit_cast(V, o[j]);
        if (redo != 0) {  // rare: an element the quick route could not settle
#pragma unroll
            for (int e = 0; e < VN; ++e)
                if (redo & (1u << e)) {
                    T a[Op::NIN], r[Op::NOUT];
#pragma unroll
                    for (int i = 0; i < Op::NIN; ++i) a[i] = Vec<T>::get(in[i][0], e);
                    op(a, r);
#pragma unroll
                    for (int j = 0; j < Op::NOUT; ++j) Vec<T>::set(res[j], e, r[j]);
                }
        }
#pragma unroll
        for (int j = 0; j < Op::NOUT; ++j)
            st<NT>(reinterpret_cast<V *>(tp.p[Op::out_slot(j)]) + v0, res[j]);
        return;
    }

    V out[Op::NOUT][UNROLL];
    static_assert(UNROLL * VN <= 32, "one redo bit per element of a lane");
    [[maybe_unused]] uint32_t redo = 0;
#pragma unroll
    for (int k = 0; k < UNROLL; ++k)
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            T a[Op::NIN], r[Op::NOUT];
#pragma unroll
            for (int i = 0; i < Op::NIN; ++i) a[i] = Vec<T>::get(in[i][k], e);
            if constexpr (IsSpeculative<Op>::value) {
                if (!op.quick(a, r)) redo |= 1u << (k * VN + e);
            } else {
                op(a, r);
            }
#pragma unroll
            for (int j = 0; j < Op::NOUT; ++j) Vec<T>::set(out[j][k], e, r[j]);
        }

    if constexpr (IsSpeculative<Op>::value) {
        if (redo != 0) {  // rare: some lane has an element the quick route could not settle
#pragma unroll
            for (int k = 0; k < UNROLL; ++k)
#pragma unroll
                for (int e = 0; e < VN; ++e)
                    if (redo & (1u << (k * VN + e))) {
                        T a[Op::NIN], r[Op::NOUT];
#pragma unroll
                        for (int i = 0; i < Op::NIN; ++i) a[i] = Vec<T>::get(in[i][k], e);
                        op(a, r);
#pragma unroll
                        for (int j = 0; j < Op::NOUT; ++j) Vec<T>::set(out[j][k], e, r[j]);
                    }
        }
    }

#pragma unroll
    for (int k = 0; k < UNROLL; ++k)
#pragma unroll
        for (int j = 0; j < Op::NOUT; ++j)
            st<NT>(reinterpret_cast<V *>(tp.p[Op::out_slot(j)]) + v0 + (size_t)k * kBlock,
                   out[j][k]);
}

// The staged schedule of a whole tile (ops with IsStaged): the op's own program of loads, waits
// and stores, one memory operation of the wave in flight at a time (two where a store and the
// next load go out together), every result stored as soon as it exists.  Same arithmetic as
// tile_full, other order of memory operations -- so the arrays of a tensor must not overlap one
// another (the host checks; tile_full loads everything before it stores).
template <typename T, class Op, bool NT, int ORDER = 0>
__device__ __forceinline__ void tile_full_staged(const Op &op, const TensorPtrs<T, Op> &tp,
                                                 size_t vec_base) {
    const StagedIO<T, Op, NT> io{tp.p, vec_base + threadIdx.x};
    if constexpr (ORDER != 0) {
        static_assert(ORDER < LoadOrders<Op>::value, "the op has no such load order");
        op.template staged_in_order<ORDER>(io);
    } else {
        op.staged(io);
    }
}

// All pointers 16-byte aligned, tile cut short by the end of the tensor:
// `rem` (< Tile::ELEMS) elements remain from element index `base`.
template <typename T, class Op, int UNROLL>
__device__ __forceinline__ void tile_partial(const Op &op, const TensorPtrs<T, Op> &tp,
                                             size_t base, uint32_t rem) {
    using V = typename Vec<T>::type;
    constexpr int VN = Vec<T>::N;
    const uint32_t nvec = rem / VN;
    const size_t vbase = base / VN;  // base is a multiple of Tile::ELEMS
    for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
        V in[Op::NIN], out[Op::NOUT];
#pragma unroll
        for (int i = 0; i < Op::NIN; ++i)
            in[i] = as_global(reinterpret_cast<const V *>(tp.p[i]))[vbase + v];
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            T a[Op::NIN], r[Op::NOUT];
#pragma unroll
            for (int i = 0; i < Op::NIN; ++i) a[i] = Vec<T>::get(in[i], e);
            op(a, r);
#pragma unroll
            for (int j = 0; j < Op::NOUT; ++j) Vec<T>::set(out[j], e, r[j]);
        }
#pragma unroll
        for (int j = 0; j < Op::NOUT; ++j)
            as_global(reinterpret_cast<V *>(tp.p[Op::out_slot(j)]))[vbase + v] = out[j];
    }
    // the last rem % VN elements, one lane each
    const uint32_t done = nvec * VN;
    if (threadIdx.x < rem - done) {
        const size_t i0 = base + done + threadIdx.x;
        T a[Op::NIN], r[Op::NOUT];
#pragma unroll
        for (int i = 0; i < Op::NIN; ++i) a[i] = ld_elem(tp.p[i], i0);
        op(a, r);
#pragma unroll
        for (int j = 0; j < Op::NOUT; ++j) st_elem(tp.p[Op::out_slot(j)], i0, r[j]);
    }
}

// Some pointer is not 16-byte aligned: element-wise accesses, still coalesced
// (consecutive lanes touch consecutive elements).
template <typename T, class Op, int UNROLL>
__device__ __forceinline__ void tile_unaligned(const Op &op, const TensorPtrs<T, Op> &tp,
                                               size_t base, uint32_t cnt) {
    constexpr int STEPS = 4;
    for (uint32_t e0 = 0; e0 < cnt; e0 += kBlock * STEPS) {
        T a[STEPS][Op::NIN];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint32_t e = e0 + s * kBlock + threadIdx.x;
            if (e < cnt) {
#pragma unroll
                for (int i = 0; i < Op::NIN; ++i) a[s][i] = ld_elem(tp.p[i], base + e);
            }
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint32_t e = e0 + s * kBlock + threadIdx.x;
            if (e < cnt) {
                T r[Op::NOUT];
                op(a[s], r);
#pragma unroll
                for (int j = 0; j < Op::NOUT; ++j) st_elem(tp.p[Op::out_slot(j)], base + e, r[j]);
            }
        }
    }
}

template <typename T, class Op>
__device__ __forceinline__ bool all_aligned16(const TensorPtrs<T, Op> &tp) {
    uintptr_t bits = 0;
#pragma unroll
    for (int i = 0; i < Op::NPTR; ++i) bits |= reinterpret_cast<uintptr_t>(tp.p[i]);
    return (bits & 15u) == 0;
}

template <typename T, class Op, int UNROLL, bool NT, bool STAGED = false>
__device__ __forceinline__ void process_tile(const Op &op, const TensorPtrs<T, Op> &tp, size_t n,
                                             size_t tile, bool aligned) {
    using TL = Tile<T, UNROLL>;
    const size_t base = tile * TL::ELEMS;
    const size_t left = n - base;
    if (aligned) {
        if (left >= (size_t)TL::ELEMS) {
            if constexpr (STAGED)
                tile_full_staged<T, Op, NT>(op, tp, tile * TL::VECS);
            else
                tile_full<T, Op, UNROLL, NT>(op, tp, tile * TL::VECS);
        } else
            tile_partial<T, Op, UNROLL>(op, tp, base, (uint32_t)left);
    } else {
        const uint32_t cnt = left >= (size_t)TL::ELEMS ? (uint32_t)TL::ELEMS : (uint32_t)left;
        tile_unaligned<T, Op, UNROLL>(op, tp, base, cnt);
    }
}

// ---------------------------------------------------------------------------
// Single-tensor kernel: one workgroup per tile (the stride loop only runs more
// than once for tensors beyond the grid limit).
// ---------------------------------------------------------------------------
template <typename T, class Op, int UNROLL, bool NT>
__global__ __launch_bounds__(kBlock) void stream_kernel(const Op op, const TensorPtrs<T, Op> tp,
                                                        const size_t n, const size_t num_tiles) {
    const bool aligned = all_aligned16<T, Op>(tp);
    const Op live = live_op(op);
    for (size_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x)
        process_tile<T, Op, UNROLL, NT>(live, tp, n, tile, aligned);
}

// The common case without its branches: every pointer 16-byte aligned and only whole tiles,
// one workgroup per tile.  The host launches this over the whole tiles of a tensor and hands a
// ragged last tile to stream_kernel.
template <typename T, class Op, int UNROLL, bool NT, bool STAGED = false, int ORDER = 0>
__global__ __launch_bounds__(kBlock) void full_tiles_kernel(const Op op,
                                                            const TensorPtrs<T, Op> tp) {
    static_assert(!STAGED || UNROLL == 1, "the staged schedule handles one vector per lane");
    static_assert(STAGED || ORDER == 0, "load orders belong to the staged schedule");
    const Op live = live_op(op);
    if constexpr (STAGED)
        tile_full_staged<T, Op, NT, ORDER>(live, tp, (size_t)blockIdx.x * Tile<T, UNROLL>::VECS);
    else
        tile_full<T, Op, UNROLL, NT>(live, tp, (size_t)blockIdx.x * Tile<T, UNROLL>::VECS);
}

// ---------------------------------------------------------------------------
// Multi-tensor kernel.  The per-tensor table travels in the kernel-argument
// segment (no device allocation, no upload, capturable in a HIP graph).  As in
// the single-tensor kernel one workgroup handles one tile, and workgroup ids
// follow the concatenation of all tensors' tiles, so the dispatcher still walks
// memory in order.
//
// A workgroup finds its tensor from its tile id in two dependent scalar loads:
// the exclusive prefix sums of tile counts are stored in groups of eight, and
// `coarse` holds the first prefix of every group but the first.  Counting the
// coarse entries <= tile picks the group (one 64-byte load), counting inside
// the group picks the tensor (one 32-byte load); a third load fetches that
// tensor's record.  Everything is wave-uniform and runs on the scalar unit
// against the scalar cache.  (A binary search costs seven dependent loads and
// measured 10 % slower end to end.)
// ---------------------------------------------------------------------------
// Bytes of kernel-argument space given to the table.  With the op's scalars
// (at most 48 bytes) and the 256 bytes of implicit arguments the whole segment
// stays under the 4 KiB HIP allows.
constexpr int kKernargBudget = 3712;
constexpr int kGroup = 8;       // prefix sums per group
constexpr int kMaxGroups = 16;  // coarse entries (one 64-byte scalar load)
constexpr uint32_t kNoTile = 0xffffffffu;

template <typename T, class Op>
struct MultiTable {
    struct Rec {  // one tensor
        T *p[Op::NPTR];
        uint64_t n;
    };
    struct alignas(32) Group {
        uint32_t start[kGroup];  // first global tile of each tensor; kNoTile past the end
    };
    static constexpr int kPerTensor = (int)sizeof(Rec) + 4;
    static constexpr int kFit = (kKernargBudget - 64 - 16) / kPerTensor / kGroup * kGroup;
    static constexpr int MAX = kFit < kGroup * kMaxGroups ? kFit : kGroup * kMaxGroups;
    static constexpr int GROUPS = MAX / kGroup;

    alignas(64) uint32_t coarse[kMaxGroups];  // coarse[g] = group[g + 1].start[0], else kNoTile
    Group group[GROUPS];
    Rec rec[MAX];
    uint32_t total;  // tiles in this launch
};

template <typename T, class Op, int UNROLL, bool NT, bool STAGED = false>
__global__ __launch_bounds__(kBlock) void multi_stream_kernel(const Op op,
                                                              const MultiTable<T, Op> tab) {
    using Table = MultiTable<T, Op>;
    const Op live = live_op(op);
    for (uint32_t tile = blockIdx.x; tile < tab.total; tile += gridDim.x) {
        uint32_t g = 0;
#pragma unroll
        for (int i = 0; i < kMaxGroups; ++i) g += (tab.coarse[i] <= tile) ? 1u : 0u;
        const typename Table::Group grp = tab.group[g];
        uint32_t k = 0;
#pragma unroll
        for (int i = 1; i < kGroup; ++i) k += (grp.start[i] <= tile) ? 1u : 0u;
        uint32_t first = grp.start[0];
#pragma unroll
        for (int i = 1; i < kGroup; ++i) first = (grp.start[i] <= tile) ? grp.start[i] : first;
        const typename Table::Rec rec = tab.rec[g * kGroup + k];
        TensorPtrs<T, Op> tp;
#pragma unroll
        for (int i = 0; i < Op::NPTR; ++i) tp.p[i] = rec.p[i];
        const bool aligned = all_aligned16<T, Op>(tp);
        process_tile<T, Op, UNROLL, NT, STAGED>(live, tp, (size_t)rec.n, (size_t)(tile - first),
                                                aligned);
    }
}

// ---------------------------------------------------------------------------
// Lists longer than a kernel-argument table: the records live in device memory (a "plan"), so
// one launch covers a list of any length.
//
// A plan is one 96-byte record per tensor.  The launch carries, in its kernel arguments, a
// coarse index: for every cell of 2^shift consecutive tiles of the global tile numbering, the
// number of the record that owns the cell's first tile.  A workgroup reads its cell's entry
// (kernel arguments: hot in the scalar cache), then that record (hot too: thousands of
// consecutive tiles share it), and has its tensor unless a tensor boundary lies in the cell
// before its tile; then it walks the records forward, at most as many steps as tensors start
// inside one cell.  Records reach the device in kernel arguments of small fill kernels (no copy
// engine, no pinned staging, nothing for a later launch to find changed).
// ---------------------------------------------------------------------------
constexpr int kPlanSlots = 9;  // most pointer slots of any op (backward_all with both gradients)

struct alignas(32) PlanRec {
    void *p[kPlanSlots];
    uint64_t n;           // elements
    uint32_t first;       // first global tile of this tensor
    uint32_t next_first;  // first global tile of the next tensor (the total for the last one)
    uint32_t index;       // position in the record array
    uint32_t reserved;
};
static_assert(sizeof(PlanRec) == 96, "three 32-byte scalar loads");

constexpr int kPlanCells = 832;  // 3328 bytes of kernel arguments

struct PlanView {
    const PlanRec *recs;
    // Lists of thousands of small tensors: 832 cells would leave dozens of records per cell for a
    // wave to walk, so such a plan carries a finer index of the same kind in device memory (one
    // entry per 2^fine_shift tiles, about two to four entries per record) and waves start from
    // that; nullptr for every other list.
    const uint32_t *fine;
    uint32_t total;       // tiles
    uint32_t shift;       // log2 of the tiles per cell
    uint32_t num;         // records
    uint32_t fine_shift;  // log2 of the tiles per entry of `fine`
    uint32_t cell[kPlanCells];  // record that owns tile (i << shift)
};

// What the host knows of one tensor, as it travels in kernel arguments.
template <int NPTR>
struct PlanSeed {
    void *p[NPTR];
    uint64_t n;
    uint32_t first, next_first;
};
template <int NPTR>
struct PlanSeedChunk {
    static constexpr int MAX = 3584 / (int)sizeof(PlanSeed<NPTR>);
    PlanSeed<NPTR> seed[MAX];
};

template <int NPTR>
__global__ __launch_bounds__(128) void plan_fill_kernel(PlanRec *recs, uint32_t at, uint32_t count,
                                                        const PlanSeedChunk<NPTR> chunk) {
    const uint32_t i = threadIdx.x;
    if (i >= count) return;
    PlanRec r;
#pragma unroll
    for (int j = 0; j < kPlanSlots; ++j) r.p[j] = nullptr;
#pragma unroll
    for (int j = 0; j < NPTR; ++j) r.p[j] = chunk.seed[i].p[j];
    r.n = chunk.seed[i].n;
    r.first = chunk.seed[i].first;
    r.next_first = chunk.seed[i].next_first;
    r.index = at + i;
    r.reserved = 0;
    recs[at + i] = r;
}
static_assert(PlanSeedChunk<kPlanSlots>::MAX >= 1 && PlanSeedChunk<3>::MAX <= 128,
              "one fill workgroup covers a chunk");

// The finer index of a plan with very many records: entry c = the record that owns tile
// c << shift, found by bisection over the records' first tiles (strictly increasing: a plan holds
// non-empty tensors only).
__global__ __launch_bounds__(256) void plan_index_kernel(const PlanRec *recs, uint32_t num,
                                                         uint32_t *fine, uint32_t entries,
                                                         uint32_t shift) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= entries) return;
    const uint32_t tile = c << shift;
    uint32_t lo = 0, hi = num - 1;  // the largest k with recs[k].first <= tile
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo + 1) / 2;
        if (recs[mid].first <= tile)
            lo = mid;
        else
            hi = mid - 1;
    }
    fine[c] = lo;
}

// A record read at a wave-uniform address from memory no kernel writes while this one runs:
// through the constant address space, so the scalar unit fetches it (three 32-byte loads).
__device__ __forceinline__ PlanRec load_record(const PlanRec *at) {
    using ConstWord = const __attribute__((address_space(4))) uint64_t;
    ConstWord *w = (ConstWord *)at;
    PlanRec r;
#pragma unroll
    for (int j = 0; j < kPlanSlots; ++j) r.p[j] = reinterpret_cast<void *>(w[j]);
    r.n = w[kPlanSlots];
    const uint64_t tiles = w[kPlanSlots + 1], rest = w[kPlanSlots + 2];
    r.first = (uint32_t)tiles;
    r.next_first = (uint32_t)(tiles >> 32);
    r.index = (uint32_t)rest;
    r.reserved = 0;
    return r;
}

template <typename T, class Op, int UNROLL, bool NT, bool STAGED = false>
__global__ __launch_bounds__(kBlock) void plan_stream_kernel(const Op op, const PlanView plan) {
    const Op live = live_op(op);
    // The records of a launch that follows other work are in no cache: left alone, the first wave
    // to need a record fetches it from memory while every wave dispatched behind it waits on the
    // same line -- a hiccup of the dispatch frontier at every tensor boundary (10-35 us over the
    // 290 tensors of a GPT-2-medium list, 1-2.5 % of the launch; a launch that follows its own kind
    // finds them in the L2s).  So the first 8 x num workgroups of the grid each touch one record
    // on their way: workgroups are dealt to the 8 XCDs in turn, so workgroups 8k .. 8k+7 put
    // record k into each XCD's L2 during the launch's first microseconds.
    if (blockIdx.x < plan.num * 8u) {
        const uint32_t *rec = reinterpret_cast<const uint32_t *>(plan.recs + (blockIdx.x >> 3));
        const uint32_t head = load_uniform(rec), tail = load_uniform(rec + sizeof(PlanRec) / 4 - 1);
        asm volatile("" ::"s"(head), "s"(tail));
    }
    // The host launches at most plan.total workgroups, so the first tile needs no bounds check:
    // a wave's first dependent fetch is its cell, not the total.
    uint32_t tile = blockIdx.x;
    do {
        const uint32_t start = plan.fine != nullptr ? load_uniform(plan.fine + (tile >> plan.fine_shift))
                                                    : plan.cell[tile >> plan.shift];
        PlanRec rec = load_record(plan.recs + start);
        // All twelve words of the record are fetched now, in one go (three 32-byte scalar loads
        // in flight together): left alone, the compiler fetches the four words the walk below
        // tests, waits, and only then fetches the pointers -- one more round trip to the scalar
        // cache in every wave's prologue.
#pragma unroll
        for (int i = 0; i < kPlanSlots; ++i) asm volatile("" : "+s"(rec.p[i]));
        // a tensor boundary lies between the cell's first tile and this one: walk on (never
        // past the last record)
        while (tile >= rec.next_first && rec.index + 1 < plan.num)
            rec = load_record(plan.recs + (rec.index + 1));
        TensorPtrs<T, Op> tp;
#pragma unroll
        for (int i = 0; i < Op::NPTR; ++i) tp.p[i] = static_cast<T *>(rec.p[i]);
        const bool aligned = all_aligned16<T, Op>(tp);
        process_tile<T, Op, UNROLL, NT, STAGED>(live, tp, (size_t)rec.n, (size_t)(tile - rec.first),
                                                aligned);
        tile += gridDim.x;
    } while (tile < plan.total);
}

// count <- count + (count != INT64_MAX): the reference's inc_count
// (/root/reference/torchopt/transform/utils.py:111-126) for a step number that lives on the device.
__global__ __launch_bounds__(64) void count_advance_kernel(int64_t *count) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        const int64_t c = *count;
        *count = c + (c != INT64_MAX ? 1 : 0);
    }
}

// Clock evidence for a measurement: one lane runs `spins` dependent integer multiply-adds and
// reports how many shader-clock ticks (s_memtime) and how many ticks of the constant-rate
// counter (s_memrealtime, 100 MHz) that took.  The ratio is the shader clock the wave ran at;
// the constant-rate ticks for a fixed spin say the same without trusting either counter's name.
__global__ __launch_bounds__(64) void clock_probe_kernel(uint64_t *out, uint32_t spins) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const uint64_t wall0 = wall_clock64();
    const uint64_t core0 = clock64();
    uint32_t x = spins | 1u;
    for (uint32_t i = 0; i < spins; ++i) {
        x = x * 1664525u + 1013904223u;
        asm volatile("" : "+v"(x));  // keeps the chain: one multiply-add after the other
    }
    const uint64_t core1 = clock64();
    const uint64_t wall1 = wall_clock64();
    out[0] = core1 - core0;
    out[1] = wall1 - wall0;
    out[2] = x;
}

}  // namespace toa
