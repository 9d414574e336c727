/*
 * CPU oracle for the fused Adam operator -- TEST INFRASTRUCTURE, NOT PRODUCT.
 * See adam_oracle.h for who may use it and how it is pinned.
 *
 * Arithmetic contract restated from
 * /root/reference/src/adam_op/adam_op_impl_cpu.cpp:
 *   - all hyper-parameters arrive as double and are rounded to the element
 *     type T before the loop (":78-84" and the other launchers);
 *   - (1 - b1), (1 - b2) are formed in T inside the loop (":51-52");
 *   - bias corrections are reciprocals formed in double, rounded to T and
 *     multiplied, never divided (":73-74, 53-54");
 *   - every product and sum is rounded separately (the reference build is
 *     -O3 on baseline x86-64: no FMA, /root/reference/CMakeLists.txt:46-48);
 *   - sqrt is the element type's own (sqrtf for float);
 *   - the tail of backward_updates multiplies by the double literal 0.5, so
 *     for float the last three products are carried in double and rounded
 *     once (":314-315").
 * Thread policy as in the reference (":30, 43-46"): OpenMP static schedule,
 * min(n/1000, nprocs) threads, serial when n <= 1000.
 *
 * Build with -ffp-contract=off (the Makefile does).
 */
#include "adam_oracle.h"

#include <math.h>
#include <omp.h>
#include <string.h>

#define MIN_N_PARALLEL 1000u

int oracle_adam_threads_for(size_t n) {
    if (n <= MIN_N_PARALLEL) return 1;
    size_t want = n / MIN_N_PARALLEL;
    size_t have = (size_t)omp_get_num_procs();
    return (int)(want < have ? want : have);
}

void oracle_adam_host_scalars(double b1, double b2, double eps_root, uint64_t count,
                              double out[4]) {
    /* std::pow(double, size_t) promotes the exponent to double. */
    const double pb1 = pow(b1, (double)count);
    const double pb2 = pow(b2, (double)count);
    out[0] = 1 / (1 - pb1);
    out[1] = 1 / (1 - pb2);
    out[2] = 1 - pb1;
    out[3] = 1 / (1 - pb2 + eps_root);
}

#define PRAGMA_(x) _Pragma(#x)
#define PAR_FOR(n) \
    PRAGMA_(omp parallel for schedule(static) num_threads(oracle_adam_threads_for(n)) if ((n) > MIN_N_PARALLEL))

#define ORACLE_DEFINE(T, SFX, SQRT)                                                            \
                                                                                               \
    void oracle_adam_forward_inplace_##SFX(T *updates, T *mu, T *nu, size_t n, double b1_,     \
                                           double b2_, double eps_, double eps_root_,          \
                                           uint64_t count) {                                   \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const T b1 = (T)b1_, b2 = (T)b2_, eps = (T)eps_, eps_root = (T)eps_root_;              \
        const T c1 = (T)s[0], c2 = (T)s[1];                                                    \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T g = updates[i], m = mu[i], v = nu[i];                                      \
            const T m1 = b1 * m + (1 - b1) * g;                                                \
            const T v1 = b2 * v + (1 - b2) * g * g;                                            \
            const T mh = m1 * c1;                                                              \
            const T vh = v1 * c2;                                                              \
            const T u1 = mh / (SQRT(vh + eps_root) + eps);                                     \
            mu[i] = m1;                                                                        \
            nu[i] = v1;                                                                        \
            updates[i] = u1;                                                                   \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_mu_##SFX(const T *updates, const T *mu, size_t n, double b1_,     \
                                      T *mu_out) {                                             \
        const T b1 = (T)b1_;                                                                   \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) mu_out[i] = b1 * mu[i] + (1 - b1) * updates[i];         \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_nu_##SFX(const T *updates, const T *nu, size_t n, double b2_,     \
                                      T *nu_out) {                                             \
        const T b2 = (T)b2_;                                                                   \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T g = updates[i];                                                            \
            nu_out[i] = b2 * nu[i] + (1 - b2) * g * g;                                         \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_updates_##SFX(const T *new_mu, const T *new_nu, size_t n,         \
                                           double b1_, double b2_, double eps_,                \
                                           double eps_root_, uint64_t count, T *updates_out) { \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const T eps = (T)eps_, eps_root = (T)eps_root_;                                        \
        const T c1 = (T)s[0], c2 = (T)s[1];                                                    \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T mh = new_mu[i] * c1;                                                       \
            const T vh = new_nu[i] * c2;                                                       \
            updates_out[i] = mh / (SQRT(vh + eps_root) + eps);                                 \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_mu_##SFX(const T *dmu, size_t n, double b1_, T *dupdates_out,    \
                                       T *dmu_out) {                                           \
        const T b1 = (T)b1_;                                                                   \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T d = dmu[i];                                                                \
            dupdates_out[i] = (1 - b1) * d;                                                    \
            dmu_out[i] = b1 * d;                                                               \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_nu_##SFX(const T *dnu, const T *updates, size_t n, double b2_,   \
                                       T *dupdates_out, T *dnu_out) {                          \
        const T b2 = (T)b2_;                                                                   \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T d = dnu[i], g = updates[i];                                                \
            dupdates_out[i] = 2 * (1 - b2) * g * d;                                            \
            dnu_out[i] = b2 * d;                                                               \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_updates_##SFX(const T *dupdates, const T *updates,               \
                                            const T *new_mu, size_t n, double b1_,             \
                                            double b2_, double eps_root_, uint64_t count,      \
                                            T *dnew_mu_out, T *dnew_nu_out) {                  \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const T p1 = (T)s[2], q2 = (T)s[3];                                                    \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T d = dupdates[i], u = updates[i], m1 = new_mu[i];                           \
            if (m1 == 0) {                                                                     \
                dnew_mu_out[i] = 0;                                                            \
                dnew_nu_out[i] = 0;                                                            \
                continue;                                                                      \
            }                                                                                  \
            const T r = u / m1;                                                                \
            const T den = r * p1;                                                              \
            dnew_mu_out[i] = d * r;                                                            \
            /* T*T, T*T, then T*double: the 0.5 literal lifts the tail to double */            \
            dnew_nu_out[i] = (T)(-d * u * den * 0.5 * q2 * den);                               \
        }                                                                                      \
    }

/* The classic in-place optimizer step as the reference chains perform it, their passes
 * restated as statements per element (element-wise, so the order of passes and elements is
 * immaterial); paths under /root/reference/torchopt:
 *   1. [maximize] g = -g                          alias/utils.py:148
 *   2. [decay == 1, adam]  g = g + wd * p         alias/utils.py:113-122
 *   3. Adam forward_ in place                     adam_op_impl_cpu.cpp:32-91
 *   4. [decay == 2, adamw] u = u + wd * p         transform/add_decayed_weights.py:232-239
 *   5. updates *= -lr (scalar rounded to T)       transform/scale.py:93-98
 *   6. params += updates                          update.py:71-74
 * Steps 2 and 4 are Tensor.add_(p, alpha=wd), which torch evaluates as one fused multiply-add
 * (a single rounding), hence fma() here.  With write_updates == 0 the updates array is left as
 * it was (the fused GPU step can skip that store); params, mu and nu are the same either way. */
#define ORACLE_DEFINE_STEP(T, SFX, SQRT, FMA)                                                  \
    void oracle_adam_fused_step_##SFX(T *params, T *updates, T *mu, T *nu, size_t n,           \
                                      double b1_, double b2_, double eps_, double eps_root_,   \
                                      uint64_t count, double lr_, double wd_, int decay,       \
                                      int maximize, int write_updates) {                       \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const T b1 = (T)b1_, b2 = (T)b2_, eps = (T)eps_, eps_root = (T)eps_root_;              \
        const T c1 = (T)s[0], c2 = (T)s[1], neg_lr = (T)(-lr_), wd = (T)wd_;                   \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            T g = maximize ? -updates[i] : updates[i];                                         \
            if (decay == 1) g = FMA(wd, params[i], g);                                         \
            const T m1 = b1 * mu[i] + (1 - b1) * g;                                            \
            const T v1 = b2 * nu[i] + (1 - b2) * g * g;                                        \
            const T mh = m1 * c1;                                                              \
            const T vh = v1 * c2;                                                              \
            T u1 = mh / (SQRT(vh + eps_root) + eps);                                           \
            if (decay == 2) u1 = FMA(wd, params[i], u1);                                       \
            const T step = u1 * neg_lr;                                                        \
            mu[i] = m1;                                                                        \
            nu[i] = v1;                                                                        \
            params[i] = params[i] + step;                                                      \
            if (write_updates) updates[i] = step;                                              \
        }                                                                                      \
    }

ORACLE_DEFINE(float, f32, sqrtf)
ORACLE_DEFINE(double, f64, sqrt)
ORACLE_DEFINE_STEP(float, f32, sqrtf, fmaf)
ORACLE_DEFINE_STEP(double, f64, sqrt, fma)


/* ---------------------------------------------------------------------------------------------
 * Half precision and bfloat16.
 *
 * The reference CPU op also dispatches at::Half and at::BFloat16 (include/common.h:26-31 with
 * USE_FP16 undefined, the default build).  The kernels are then instantiated with scalar_t =
 * c10::Half / c10::BFloat16, whose arithmetic is: convert both operands to float, operate in
 * float, and -- when both operands are the 16-bit type (or an int, which converts to it first) --
 * round the result back to 16 bits; an operation between the 16-bit type and a float (double)
 * yields a float (double) that is not rounded.  Consequences for adam_op_impl_cpu.cpp:
 *   - every product, sum and difference in the moment updates is rounded to 16 bits;
 *   - sqrt(nu_hat + eps_root) is the float overload applied to the 16-bit sum, so the square
 *     root, "+ eps" and the division run in float and only the quotient is rounded (":59");
 *   - the tail of backward_updates runs in double after two 16-bit products, and the result
 *     goes double -> float -> 16 bits (":314-315");
 *   - every scalar goes double -> float -> 16 bits (":78-84").
 * Values are kept as float holding an exactly representable 16-bit value; RND() rounds a float
 * to the format and back.  Storage is uint16_t bit patterns.
 * ------------------------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float f32_from(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary16 <- binary32, round to nearest even; NaN -> sign | 0x7e00. */
static inline uint16_t f16_from_f32(float f) {
    const uint32_t x = f32_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t a = x & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to infinity */
    if (a < 0x38800000u) {                                   /* below 2^-14: subnormal or zero */
        /* units of 2^-24; exact product, then one round-to-nearest-even to an integer */
        const float units = nearbyintf(f32_from(a) * 0x1p24f);
        return (uint16_t)(sign | (uint16_t)units);
    }
    uint32_t h = (((a >> 23) - 112u) << 10) | ((a & 0x7fffffu) >> 13);
    const uint32_t rest = a & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) ++h; /* carry may bump the exponent */
    return (uint16_t)(sign | h);
}

static inline float f32_from_f16(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) {
        const float mag = (float)m * 0x1p-24f;
        return sign ? -mag : mag;
    }
    if (e == 31) return f32_from(sign | 0x7f800000u | (m << 13));
    return f32_from(sign | ((e + 112u) << 23) | (m << 13));
}

/* bfloat16 <- binary32: round to nearest even on the upper 16 bits; NaN -> 0x7fc0. */
static inline uint16_t bf16_from_f32(float f) {
    const uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}
static inline float f32_from_bf16(uint16_t b) { return f32_from((uint32_t)b << 16); }

#define ORACLE_DEFINE_LOWP(SFX, TO16, FROM16)                                                  \
    static inline float rnd_##SFX(float x) { return FROM16(TO16(x)); }                         \
                                                                                               \
    void oracle_adam_forward_inplace_##SFX(uint16_t *updates, uint16_t *mu, uint16_t *nu,      \
                                           size_t n, double b1_, double b2_, double eps_,      \
                                           double eps_root_, uint64_t count) {                 \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const float b1 = rnd_##SFX((float)b1_), b2 = rnd_##SFX((float)b2_);                    \
        const float eps = rnd_##SFX((float)eps_), er = rnd_##SFX((float)eps_root_);            \
        const float c1 = rnd_##SFX((float)s[0]), c2 = rnd_##SFX((float)s[1]);                  \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float g = FROM16(updates[i]), m = FROM16(mu[i]), v = FROM16(nu[i]);          \
            const float m1 =                                                                   \
                rnd_##SFX(rnd_##SFX(b1 * m) + rnd_##SFX(rnd_##SFX(1.0f - b1) * g));            \
            const float v1 = rnd_##SFX(                                                        \
                rnd_##SFX(b2 * v) + rnd_##SFX(rnd_##SFX(rnd_##SFX(1.0f - b2) * g) * g));       \
            const float mh = rnd_##SFX(m1 * c1), vh = rnd_##SFX(v1 * c2);                      \
            const float u1 = mh / (sqrtf(rnd_##SFX(vh + er)) + eps);                           \
            mu[i] = TO16(m1);                                                                  \
            nu[i] = TO16(v1);                                                                  \
            updates[i] = TO16(u1);                                                             \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_mu_##SFX(const uint16_t *updates, const uint16_t *mu, size_t n,   \
                                      double b1_, uint16_t *mu_out) {                          \
        const float b1 = rnd_##SFX((float)b1_);                                                \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i)                                                         \
            mu_out[i] = TO16(rnd_##SFX(b1 * FROM16(mu[i])) +                                   \
                             rnd_##SFX(rnd_##SFX(1.0f - b1) * FROM16(updates[i])));            \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_nu_##SFX(const uint16_t *updates, const uint16_t *nu, size_t n,   \
                                      double b2_, uint16_t *nu_out) {                          \
        const float b2 = rnd_##SFX((float)b2_);                                                \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float g = FROM16(updates[i]);                                                \
            nu_out[i] = TO16(rnd_##SFX(b2 * FROM16(nu[i])) +                                   \
                             rnd_##SFX(rnd_##SFX(rnd_##SFX(1.0f - b2) * g) * g));              \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_forward_updates_##SFX(const uint16_t *new_mu, const uint16_t *new_nu,     \
                                           size_t n, double b1_, double b2_, double eps_,      \
                                           double eps_root_, uint64_t count,                   \
                                           uint16_t *updates_out) {                            \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const float eps = rnd_##SFX((float)eps_), er = rnd_##SFX((float)eps_root_);            \
        const float c1 = rnd_##SFX((float)s[0]), c2 = rnd_##SFX((float)s[1]);                  \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float mh = rnd_##SFX(FROM16(new_mu[i]) * c1);                                \
            const float vh = rnd_##SFX(FROM16(new_nu[i]) * c2);                                \
            updates_out[i] = TO16(mh / (sqrtf(rnd_##SFX(vh + er)) + eps));                     \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_mu_##SFX(const uint16_t *dmu, size_t n, double b1_,              \
                                       uint16_t *dupdates_out, uint16_t *dmu_out) {            \
        const float b1 = rnd_##SFX((float)b1_);                                                \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float d = FROM16(dmu[i]);                                                    \
            dupdates_out[i] = TO16(rnd_##SFX(1.0f - b1) * d);                                  \
            dmu_out[i] = TO16(b1 * d);                                                         \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_nu_##SFX(const uint16_t *dnu, const uint16_t *updates, size_t n, \
                                       double b2_, uint16_t *dupdates_out,                     \
                                       uint16_t *dnu_out) {                                    \
        const float b2 = rnd_##SFX((float)b2_);                                                \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float d = FROM16(dnu[i]), g = FROM16(updates[i]);                            \
            dupdates_out[i] =                                                                  \
                TO16(rnd_##SFX(rnd_##SFX(2.0f * rnd_##SFX(1.0f - b2)) * g) * d);               \
            dnu_out[i] = TO16(b2 * d);                                                         \
        }                                                                                      \
    }                                                                                          \
                                                                                               \
    void oracle_adam_backward_updates_##SFX(const uint16_t *dupdates, const uint16_t *updates, \
                                            const uint16_t *new_mu, size_t n, double b1_,      \
                                            double b2_, double eps_root_, uint64_t count,      \
                                            uint16_t *dnew_mu_out, uint16_t *dnew_nu_out) {    \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const float p1 = rnd_##SFX((float)s[2]), q2 = rnd_##SFX((float)s[3]);                  \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float d = FROM16(dupdates[i]), u = FROM16(updates[i]);                       \
            const float m1 = FROM16(new_mu[i]);                                                \
            if (m1 == 0) {                                                                     \
                dnew_mu_out[i] = 0;                                                            \
                dnew_nu_out[i] = 0;                                                            \
                continue;                                                                      \
            }                                                                                  \
            const float r = rnd_##SFX(u / m1);                                                 \
            const float den = rnd_##SFX(r * p1);                                               \
            dnew_mu_out[i] = TO16(d * r);                                                      \
            const float head = rnd_##SFX(rnd_##SFX(-d * u) * den);                             \
            const double tail = (double)head * 0.5 * (double)q2 * (double)den;                 \
            dnew_nu_out[i] = TO16((float)tail);                                                \
        }                                                                                      \
    }

ORACLE_DEFINE_LOWP(f16, f16_from_f32, f32_from_f16)
ORACLE_DEFINE_LOWP(bf16, bf16_from_f32, f32_from_bf16)

/* The classic in-place optimizer step on 16-bit tensors, WITHOUT weight decay: the chain of
 * ORACLE_DEFINE_STEP above with forward_ as the low-precision restatement, and the torch calls
 * around it as torch evaluates them on 16-bit CPU tensors: Tensor.mul_(-lr) widens the tensor
 * operand to float, takes the Python scalar double -> float (NOT rounded to 16 bits), multiplies
 * in float and rounds the product to 16 bits; Tensor.add_(u) is a float addition rounded to 16
 * bits; neg_ is exact.
 * Weight decay is left out on purpose: Tensor.add_(p, alpha=wd) on 16-bit CPU tensors has no
 * single arithmetic to restate -- its vectorized body rounds alpha to 16 bits and then works in
 * float, its scalar tails (the last elements of every thread's chunk) round the product to 16
 * bits first, so an element's result depends on where it lies in the tensor.  `decay` must be 0;
 * any other value leaves the arrays untouched and returns -1. */
#define ORACLE_DEFINE_LOWP_STEP(SFX, TO16, FROM16)                                             \
    int oracle_adam_fused_step_##SFX(uint16_t *params, uint16_t *updates, uint16_t *mu,        \
                                     uint16_t *nu, size_t n, double b1_, double b2_,           \
                                     double eps_, double eps_root_, uint64_t count,            \
                                     double lr_, double wd_, int decay, int maximize,          \
                                     int write_updates) {                                      \
        (void)wd_;                                                                             \
        if (decay != 0) return -1;                                                             \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const float b1 = rnd_##SFX((float)b1_), b2 = rnd_##SFX((float)b2_);                    \
        const float eps = rnd_##SFX((float)eps_), er = rnd_##SFX((float)eps_root_);            \
        const float c1 = rnd_##SFX((float)s[0]), c2 = rnd_##SFX((float)s[1]);                  \
        const float neg_lr = (float)(-lr_);                                                    \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const float p = FROM16(params[i]), m = FROM16(mu[i]), v = FROM16(nu[i]);           \
            float g = FROM16(updates[i]);                                                      \
            if (maximize) g = -g;                                                              \
            const float m1 =                                                                   \
                rnd_##SFX(rnd_##SFX(b1 * m) + rnd_##SFX(rnd_##SFX(1.0f - b1) * g));            \
            const float v1 = rnd_##SFX(                                                        \
                rnd_##SFX(b2 * v) + rnd_##SFX(rnd_##SFX(rnd_##SFX(1.0f - b2) * g) * g));       \
            const float mh = rnd_##SFX(m1 * c1), vh = rnd_##SFX(v1 * c2);                      \
            const float u1 = rnd_##SFX(mh / (sqrtf(rnd_##SFX(vh + er)) + eps));                \
            const float step = rnd_##SFX(u1 * neg_lr);                                         \
            mu[i] = TO16(m1);                                                                  \
            nu[i] = TO16(v1);                                                                  \
            params[i] = TO16(p + step);                                                        \
            if (write_updates) updates[i] = TO16(step);                                        \
        }                                                                                      \
        return 0;                                                                              \
    }

ORACLE_DEFINE_LOWP_STEP(f16, f16_from_f32, f32_from_f16)
ORACLE_DEFINE_LOWP_STEP(bf16, bf16_from_f32, f32_from_bf16)

/* conversions, exported so tests can pin them against NumPy's float16 and torch's bfloat16 */
uint16_t oracle_f16_from_f32(float f) { return f16_from_f32(f); }
float oracle_f32_from_f16(uint16_t h) { return f32_from_f16(h); }
uint16_t oracle_bf16_from_f32(float f) { return bf16_from_f32(f); }
float oracle_f32_from_bf16(uint16_t b) { return f32_from_bf16(b); }
