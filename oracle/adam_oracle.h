/*
 * CPU oracle for the fused Adam operator -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A plain-C restatement of the reference CPU op
 * (/root/reference/src/adam_op/adam_op_impl_cpu.cpp).  Only tests, the smoke
 * check and the CPU-baseline leg of the benchmark may link or load it; the
 * shipped operator never calls into this library.
 *
 * Every function takes raw host pointers, the element count, the Python-level
 * hyper-parameters as double and `count` as an unsigned 64-bit step number --
 * the same arguments the reference's launchers receive -- and derives the
 * bias-correction scalars itself, in double, before casting to the element
 * type, as the reference does.
 *
 * Pinning status (what each function has been checked against):
 *   every function, f32 and f64: bit-for-bit against the reference's own
 *   compiled CPU op on seeded and edge-case inputs (tests/golden fixtures,
 *   written by tests/golden/make_golden.py), and against an independent
 *   NumPy one-rounding-per-operation specification (oracle/adam_spec.py);
 *   plus closed forms in tests/test_oracle.py;
 *   oracle_adam_fused_step_*: bit-for-bit against the reference chain itself run
 *   on CPU -- the compiled reference forward_ followed by the two torch calls the
 *   reference makes (Tensor.add_(p, alpha=wd), Tensor.mul_(-lr), Tensor.add_) -- in
 *   tests/test_oracle.py.
 *   No function is "parity unpinned".
 */
#ifndef ADAM_ORACLE_H
#define ADAM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* adamForwardInplaceCPU, adam_op_impl_cpu.cpp:32-91 */
void oracle_adam_forward_inplace_f32(float *updates, float *mu, float *nu, size_t n,
                                     double b1, double b2, double eps, double eps_root,
                                     uint64_t count);
void oracle_adam_forward_inplace_f64(double *updates, double *mu, double *nu, size_t n,
                                     double b1, double b2, double eps, double eps_root,
                                     uint64_t count);

/* adamForwardMuCPU, adam_op_impl_cpu.cpp:93-125 */
void oracle_adam_forward_mu_f32(const float *updates, const float *mu, size_t n, double b1,
                                float *mu_out);
void oracle_adam_forward_mu_f64(const double *updates, const double *mu, size_t n, double b1,
                                double *mu_out);

/* adamForwardNuCPU, adam_op_impl_cpu.cpp:127-160 */
void oracle_adam_forward_nu_f32(const float *updates, const float *nu, size_t n, double b2,
                                float *nu_out);
void oracle_adam_forward_nu_f64(const double *updates, const double *nu, size_t n, double b2,
                                double *nu_out);

/* adamForwardUpdatesCPU, adam_op_impl_cpu.cpp:162-209 */
void oracle_adam_forward_updates_f32(const float *new_mu, const float *new_nu, size_t n,
                                     double b1, double b2, double eps, double eps_root,
                                     uint64_t count, float *updates_out);
void oracle_adam_forward_updates_f64(const double *new_mu, const double *new_nu, size_t n,
                                     double b1, double b2, double eps, double eps_root,
                                     uint64_t count, double *updates_out);

/* adamBackwardMuCPU, adam_op_impl_cpu.cpp:211-245 */
void oracle_adam_backward_mu_f32(const float *dmu, size_t n, double b1, float *dupdates_out,
                                 float *dmu_out);
void oracle_adam_backward_mu_f64(const double *dmu, size_t n, double b1, double *dupdates_out,
                                 double *dmu_out);

/* adamBackwardNuCPU, adam_op_impl_cpu.cpp:247-284 */
void oracle_adam_backward_nu_f32(const float *dnu, const float *updates, size_t n, double b2,
                                 float *dupdates_out, float *dnu_out);
void oracle_adam_backward_nu_f64(const double *dnu, const double *updates, size_t n, double b2,
                                 double *dupdates_out, double *dnu_out);

/* adamBackwardUpdatesCPU, adam_op_impl_cpu.cpp:286-347 */
void oracle_adam_backward_updates_f32(const float *dupdates, const float *updates,
                                      const float *new_mu, size_t n, double b1, double b2,
                                      double eps_root, uint64_t count, float *dnew_mu_out,
                                      float *dnew_nu_out);
void oracle_adam_backward_updates_f64(const double *dupdates, const double *updates,
                                      const double *new_mu, size_t n, double b1, double b2,
                                      double eps_root, uint64_t count, double *dnew_mu_out,
                                      double *dnew_nu_out);

/* The reference chains' classic in-place step: [negate], [g += wd*p (decay 1)], Adam forward_,
 * [u += wd*p (decay 2)], updates *= -lr, params += updates (alias/utils.py:113-122,148,
 * adam_op_impl_cpu.cpp:32-91, transform/add_decayed_weights.py:232-239, transform/scale.py:93-98,
 * update.py:71-74). */
void oracle_adam_fused_step_f32(float *params, float *updates, float *mu, float *nu, size_t n,
                                double b1, double b2, double eps, double eps_root,
                                uint64_t count, double lr, double weight_decay, int decay,
                                int maximize, int write_updates);
void oracle_adam_fused_step_f64(double *params, double *updates, double *mu, double *nu, size_t n,
                                double b1, double b2, double eps, double eps_root,
                                uint64_t count, double lr, double weight_decay, int decay,
                                int maximize, int write_updates);
/* ... on float16 / bfloat16 bit patterns, without weight decay (`decay` must be 0, else -1 and
 * nothing is touched: torch's add_(p, alpha=wd) on 16-bit CPU tensors is not one arithmetic, see
 * the .c file): forward_ with the per-operation rounding of the 16-bit types; mul_(-lr) in float
 * with the scalar unrounded, add_ in float, one rounding to 16 bits per call.  Pinned against
 * those very calls on 16-bit CPU tensors.  Returns 0. */
int oracle_adam_fused_step_f16(uint16_t *params, uint16_t *updates, uint16_t *mu, uint16_t *nu,
                               size_t n, double b1, double b2, double eps, double eps_root,
                               uint64_t count, double lr, double weight_decay, int decay,
                               int maximize, int write_updates);
int oracle_adam_fused_step_bf16(uint16_t *params, uint16_t *updates, uint16_t *mu, uint16_t *nu,
                                size_t n, double b1, double b2, double eps, double eps_root,
                                uint64_t count, double lr, double weight_decay, int decay,
                                int maximize, int write_updates);

/* Host-side bias-correction scalars in double, before the cast to the element
 * type (adam_op_impl_cpu.cpp:73-74, 191-192, 328-329).
 *   out[0] = 1 / (1 - b1^count)              out[1] = 1 / (1 - b2^count)
 *   out[2] = 1 - b1^count                    out[3] = 1 / (1 - b2^count + eps_root) */
void oracle_adam_host_scalars(double b1, double b2, double eps_root, uint64_t count,
                              double out[4]);

/* Number of OpenMP threads the reference's policy picks for n elements
 * (adam_op_impl_cpu.cpp:30, 43-46): 1 if n <= 1000, else min(n/1000, nprocs). */
int oracle_adam_threads_for(size_t n);

#ifdef __cplusplus
}
#endif
#endif /* ADAM_ORACLE_H */
