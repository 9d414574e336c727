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

/* The classic in-place optimizer step as the reference chain performs it, three
 * passes restated as three statements per element (element-wise, so the order of
 * passes and elements is immaterial):
 *   1. [maximize] g = -g                 /root/reference/torchopt/alias/utils.py:148
 *   2. Adam forward_ in place            adam_op_impl_cpu.cpp:32-91
 *   3. updates *= -lr (scalar rounded to T)  /root/reference/torchopt/transform/scale.py:93-98
 *   4. params += updates                 /root/reference/torchopt/update.py:71-74
 * With write_updates == 0 the updates array is left as it was (the fused GPU
 * step can skip that store); params, mu and nu are the same either way. */
#define ORACLE_DEFINE_STEP(T, SFX, SQRT)                                                       \
    void oracle_adam_fused_step_##SFX(T *params, T *updates, T *mu, T *nu, size_t n,           \
                                      double b1_, double b2_, double eps_, double eps_root_,   \
                                      uint64_t count, double lr_, int maximize,                \
                                      int write_updates) {                                     \
        double s[4];                                                                           \
        oracle_adam_host_scalars(b1_, b2_, eps_root_, count, s);                               \
        const T b1 = (T)b1_, b2 = (T)b2_, eps = (T)eps_, eps_root = (T)eps_root_;              \
        const T c1 = (T)s[0], c2 = (T)s[1], neg_lr = (T)(-lr_);                                \
        PAR_FOR(n)                                                                             \
        for (size_t i = 0; i < n; ++i) {                                                       \
            const T g = maximize ? -updates[i] : updates[i];                                   \
            const T m1 = b1 * mu[i] + (1 - b1) * g;                                            \
            const T v1 = b2 * nu[i] + (1 - b2) * g * g;                                        \
            const T mh = m1 * c1;                                                              \
            const T vh = v1 * c2;                                                              \
            const T u1 = mh / (SQRT(vh + eps_root) + eps);                                     \
            const T step = u1 * neg_lr;                                                        \
            mu[i] = m1;                                                                        \
            nu[i] = v1;                                                                        \
            params[i] = params[i] + step;                                                      \
            if (write_updates) updates[i] = step;                                              \
        }                                                                                      \
    }

ORACLE_DEFINE(float, f32, sqrtf)
ORACLE_DEFINE(double, f64, sqrt)
ORACLE_DEFINE_STEP(float, f32, sqrtf)
ORACLE_DEFINE_STEP(double, f64, sqrt)
