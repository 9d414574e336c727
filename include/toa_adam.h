/*
 * toa_adam.h -- C ABI of the MI355X (gfx950) fused Adam operator library
 * (libtoa_adam.so).
 *
 * This is the boundary a host binding attaches to: plain device pointers,
 * element counts, the Python-level hyper-parameters as double, the step
 * number as an unsigned 64-bit integer and an opaque HIP stream.  No torch
 * types appear.  Each entry point replaces one device launcher of the
 * reference (declared in /root/reference/include/adam_op/adam_op_impl_cuda.cuh,
 * dispatched from /root/reference/src/adam_op/adam_op.cpp) with the tensors
 * replaced by (pointer, n, dtype).
 *
 * Conventions
 *   dtype     one of the TOA_F* codes below; all arrays of one call share it.
 *   pointers  device memory on the CURRENT HIP device, contiguous, n elements
 *             each.  Any alignment is accepted; 16-byte aligned pointers take
 *             the 128-bit path.  In toa_adam_forward_inplace the three arrays
 *             may alias one another completely (the reference's availability
 *             probe does that with n = 1).
 *   scalars   b1, b2, eps, eps_root arrive as double and are rounded to the
 *             element type inside the library; the bias corrections
 *             1/(1-b^count) etc. are formed in double first and then rounded,
 *             exactly as the reference launchers do.
 *   stream    a hipStream_t passed as void*; NULL is the device's null stream.
 *             Calls only enqueue work; they never synchronise.
 *   n == 0    is a successful no-op (no launch).
 *   return    0 on success; a positive value is a hipError_t from the launch;
 *             a negative value is one of the TOA_E* argument errors below.
 *             toa_adam_error_string() names either kind.
 *   threads   re-entrant.  Global state: the tuning knobs below and the cache of list plans (see
 *             toa_adam_set_plan_mode), which one mutex guards from the lookup until the launch
 *             that reads the plan is enqueued -- list calls from several host threads therefore
 *             take turns for the few microseconds that enqueueing costs.
 */
#ifndef TOA_ADAM_H
#define TOA_ADAM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TOA_API __attribute__((visibility("default")))

/* Element types.  TOA_F16 (IEEE half) and TOA_BF16 (bfloat16) follow the arithmetic the
 * reference CPU op performs on at::Half / at::BFloat16 tensors: every operation between two
 * 16-bit values is rounded back to 16 bits, the square root and division of the update run in
 * float and are rounded once.  The fused optimizer step takes weight decay for TOA_F32 / TOA_F64 only. */
enum { TOA_F32 = 0, TOA_F64 = 1, TOA_F16 = 2, TOA_BF16 = 3 };

enum {
    TOA_EDTYPE = -1, /* dtype not served by this entry point      */
    TOA_ENULL = -2,  /* a required pointer is NULL while n > 0    */
    TOA_ESIZE = -3,  /* a tensor is too large for the launch grid */
    TOA_ELIMIT = -4  /* beyond a stated limit of the allocation-free entry point */
};

/* Library ABI version (bumped on any signature change). */
TOA_API int toa_adam_abi_version(void);

/* Tuning knob: how many single-wave workgroups of these kernels may be resident
 * on one compute unit.  The kernels are HBM-bound and run fastest with a bounded
 * number of bytes in flight; each op has its own measured default (18 for the
 * in-place step in its staged schedule, 12 in the plain one, 16-32 for the
 * out-of-place ops).  2..32 overrides the default
 * of every op, anything else restores the per-op defaults.  The cap works
 * through LDS granules, so the levels that exist are 32, 25, 21, 18, 16, 14,
 * 12, 11, 10, 9, 8 ...; a value in between selects the next level below it.  The environment
 * variable TOA_ADAM_WAVES_PER_CU sets the initial override.  Returns the
 * previous override (0 = none).  No counterpart in the reference. */
TOA_API int toa_adam_set_waves_per_cu(int waves);

/* Tuning knob: order of a wave's memory operations in the in-place step.  The staged order is
 * load g | load mu | store mu', load nu | store nu', store u' (one memory operation of a wave
 * at a time); the plain order is all loads, then all stores.  Results are identical bit for
 * bit; only throughput differs: staged is 1.5-2 % faster on large single tensors and 12 % faster
 * where a tensor's arrays lie a multiple of 16 MiB apart and so meet in the same DRAM banks.
 *   0 (default)  single tensors staged; lists staged when a quarter of their elements belong
 *                to tensors whose arrays collide that way;
 *   1            never staged;
 *   2            staged wherever it is legal.
 * Staged needs the arrays of a tensor to be disjoint, 16-byte aligned and large enough to be
 * bandwidth-bound; other calls take the plain order whatever the setting.  (All four element
 * types have a staged form; lists of the 16-bit types run staged by default.)
 * Returns the previous setting.  No counterpart in the reference. */
TOA_API int toa_adam_set_schedule(int schedule);

/* Tuning knob: load order of the staged in-place step on one large tensor.  The staged program
 * handles the gradient and the two moments one memory operation at a time; which moment goes
 * first, and whether it is loaded before the gradient, does not change a bit of the result but
 * moves the rate by up to 1 % with where the three arrays lie:
 *   0  g | mu | store mu', nu | store nu', store u'      2  mu | g | store mu', nu | ...
 *   1  g | nu | store nu', mu | store mu', store u'      3  nu | g | store nu', mu | ...
 *  -1  (default) the library's choice.
 * The 16-bit types, lists and the other ops have one order; the setting is ignored there.
 * Returns the previous setting.  No counterpart in the reference.
 *
 * The library's choice is made per call site -- the in-place step on one set of three arrays of
 * one length, 64 MiB or more each -- by measurement on the caller's own launches: the first 30
 * launches of a site go round the four orders and the plain schedule (all loads, then all stores;
 * same bits every time), timed with events on the
 * caller's stream that are polled, never waited for; rounds alternate their direction and the
 * first two do not count, so a drift of the machine's rate cancels.  The fastest variant is kept if
 * it beats order 0 by more than 0.4 % (four samples an order cannot tell smaller differences from noise), order 0 otherwise.  On most placements order 0 wins; on
 * some another gains 1-2 %.  Up to 64 call sites are remembered.  Nothing is tuned under stream
 * capture, with an order or a residency level forced, or with a schedule other than 0.
 *   toa_adam_set_tuning         0 = every site runs order 0; 1 (default; the environment variable
 *                               TOA_ADAM_TUNING=0 starts with 0) = as above.  Returns the previous
 *                               setting.
 *   toa_adam_tuned_load_order   what was kept for that call site of toa_adam_forward_inplace: 0-3
 *                               an order of the staged program, 4 the plain schedule, -1 while
 *                               it is unknown or still being explored (the _devcount form of
 *                               the step keeps sites of its own). */
TOA_API int toa_adam_set_load_order(int order);
TOA_API int toa_adam_set_tuning(int on);
TOA_API int toa_adam_tuned_load_order(int dtype, const void *updates, const void *mu,
                                      const void *nu, size_t n);

/* Lists longer than one kernel-argument table (96 tensors for ops with three pointer slots, 80
 * with four, 64 with five, fewer beyond), and lists of 256 MiB or more per array whatever their
 * length, run as ONE launch over a device-resident table, a
 * "plan": one 96-byte record per tensor, written by small kernels that carry the records in
 * their arguments and cached per (device, stream, list) in memory the library allocates (at most
 * 16 plans per stream, 128 per process), with a coarse index from tiles to records in the launch's
 * own arguments (and, for lists of more than 1664 tensors, a finer one beside the records).  A call whose list is cached costs one launch and no other device work, and a
 * call whose arguments repeat the previous call's byte for byte (same arrays, same sizes, one step
 * count for all) skips the per-tensor host work as well: a few microseconds whatever the length.
 * Under stream capture, or when no plan memory can be had, such lists take one launch per
 * table instead (every launch then carries its table in its arguments, so a captured graph
 * depends on nothing a later call may rewrite).
 *   toa_adam_set_plan_mode   0 (default) as above; 1 never use plans; 2 use plans for every
 *                            list, however short.  Returns the previous mode.
 *   toa_adam_release_plans   frees every cached plan (waits for the devices that hold one to
 *                            drain).  Returns 0 or the last hipError_t.
 * No counterpart in the reference. */
TOA_API int toa_adam_set_plan_mode(int mode);
TOA_API int toa_adam_release_plans(void);

/* Cap on workgroups per launch (default and maximum 2^25).  Every kernel normally runs one
 * workgroup per 1 KiB tile; beyond the cap workgroups stride over the remaining tiles.  Lowering
 * the cap exercises that path on small inputs (tests) and trades dispatch work for loop
 * iterations.  0 or an out-of-range value restores the default.  Returns the previous cap.
 * No counterpart in the reference. */
TOA_API unsigned toa_adam_set_max_grid(unsigned workgroups);

/* Where to put optimizer state.  The in-place step streams three arrays at once, and how their
 * addresses fall on the memory channels moves its rate by up to 3 %.  Measured on the float32
 * step over 2^28 elements: with the two moments of a tensor 8 KiB apart modulo 16 KiB the step
 * streams at 6.80-6.87 TB/s whatever the gradient's own phase; with both at one phase it ranges
 * from 6.72 to 6.86 with the gradient's phase (an allocator hands out large blocks on 2 MiB
 * boundaries, so left alone all three arrays share their address modulo 16 KiB: 6.74-6.79).  The
 * caller owns every allocation, so this is advice in callable form:
 *   toa_adam_state_slack   extra bytes to allocate for a state array (16 KiB);
 *   toa_adam_state_shift   bytes (a multiple of 256, less than the slack) to skip from the start
 *                          of such an allocation so that the array begins at the preferred phase
 *                          of its kind: moment 0 (mu) 8 KiB past a multiple of 16 KiB, moment 1
 *                          (nu) at a multiple of 16 KiB.
 * No counterpart in the reference (its init_fn calls zeros_like,
 * /root/reference/torchopt/transform/scale_by_adam.py:401-414). */
TOA_API size_t toa_adam_state_slack(void);
TOA_API size_t toa_adam_state_shift(const void *allocation, int moment);

/* Measurement aid: enqueues a one-lane kernel on `stream` that runs `spins` (at most 2^28)
 * dependent integer multiply-adds and writes three 64-bit words to device memory at `out`: the
 * shader-clock ticks the spin took, the ticks of the device's constant-rate counter (100 MHz)
 * over the same span, and the spin's result.  ticks / constant ticks * 100 MHz is the shader
 * clock the wave ran at -- what a benchmark records beside its timings to show the clock state
 * they were taken in.  No counterpart in the reference. */
TOA_API int toa_adam_clock_probe(uint64_t *out, uint32_t spins, void *stream);

/* Human-readable name of a return code from any function below. */
TOA_API const char *toa_adam_error_string(int code);

/* ---- single-tensor entry points ---------------------------------------- */

/* Fused in-place step: mu, nu and updates are read once and overwritten.
 * Replaces adamForwardInplaceCUDA (adam_op_impl_cuda.cuh:26-33, called from
 * adam_op.cpp:41-43; arithmetic contract adam_op_impl_cpu.cpp:32-91). */
TOA_API int toa_adam_forward_inplace(int dtype, void *updates, void *mu, void *nu, size_t n, double b1,
                             double b2, double eps, double eps_root, uint64_t count,
                             void *stream);

/* mu_out = b1*mu + (1-b1)*updates.  Replaces adamForwardMuCUDA
 * (adam_op_impl_cuda.cuh:35-37, adam_op.cpp:56-58; adam_op_impl_cpu.cpp:93-125). */
TOA_API int toa_adam_forward_mu(int dtype, const void *updates, const void *mu, size_t n, double b1,
                        void *mu_out, void *stream);

/* nu_out = b2*nu + (1-b2)*updates^2.  Replaces adamForwardNuCUDA
 * (adam_op_impl_cuda.cuh:39-41, adam_op.cpp:71-73; adam_op_impl_cpu.cpp:127-160). */
TOA_API int toa_adam_forward_nu(int dtype, const void *updates, const void *nu, size_t n, double b2,
                        void *nu_out, void *stream);

/* updates_out = mu_hat / (sqrt(nu_hat + eps_root) + eps).  Replaces
 * adamForwardUpdatesCUDA (adam_op_impl_cuda.cuh:43-49, adam_op.cpp:90-92;
 * adam_op_impl_cpu.cpp:162-209). */
TOA_API int toa_adam_forward_updates(int dtype, const void *new_mu, const void *new_nu, size_t n,
                             double b1, double b2, double eps, double eps_root, uint64_t count,
                             void *updates_out, void *stream);

/* dupdates_out = (1-b1)*dmu, dmu_out = b1*dmu.  Replaces adamBackwardMuCUDA
 * (adam_op_impl_cuda.cuh:51-54, adam_op.cpp:106-108; adam_op_impl_cpu.cpp:211-245). */
TOA_API int toa_adam_backward_mu(int dtype, const void *dmu, size_t n, double b1, void *dupdates_out,
                         void *dmu_out, void *stream);

/* dupdates_out = 2*(1-b2)*updates*dnu, dnu_out = b2*dnu.  Replaces
 * adamBackwardNuCUDA (adam_op_impl_cuda.cuh:56-59, adam_op.cpp:122-124;
 * adam_op_impl_cpu.cpp:247-284). */
TOA_API int toa_adam_backward_nu(int dtype, const void *dnu, const void *updates, size_t n, double b2,
                         void *dupdates_out, void *dnu_out, void *stream);

/* Reference's hand-derived VJP of forward_updates; `updates` is the forward
 * OUTPUT.  Replaces adamBackwardUpdatesCUDA (adam_op_impl_cuda.cuh:61-68,
 * adam_op.cpp:142-145; adam_op_impl_cpu.cpp:286-347). */
TOA_API int toa_adam_backward_updates(int dtype, const void *dupdates, const void *updates,
                              const void *new_mu, size_t n, double b1, double b2,
                              double eps_root, uint64_t count, void *dnew_mu_out,
                              void *dnew_nu_out, void *stream);

/* ---- multi-tensor entry points ------------------------------------------
 * One call covers a whole list of tensors (a flattened pytree): the host loop
 * the reference runs per leaf (/root/reference/torchopt/transform/
 * scale_by_adam.py:325-332, 378-385) collapses into one launch per group of
 * tensors that share a step count (see toa_adam_set_plan_mode for long lists).  The arrays of
 * pointers, lengths and counts are HOST arrays of num_tensors entries; they
 * are consumed before the call returns.  counts may be NULL when count_all
 * applies to every tensor.  Zero-length tensors are skipped. */

TOA_API int toa_adam_forward_inplace_multi(int dtype, size_t num_tensors, void *const *updates,
                                   void *const *mu, void *const *nu, const size_t *n, double b1,
                                   double b2, double eps, double eps_root,
                                   const uint64_t *counts, uint64_t count_all, void *stream);

/* toa_adam_forward_inplace_multi for callers that cannot allocate device memory -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments, same results bit for bit, always one launch per distinct step
 * count however long the list; the per-tensor records live in a device array built into the
 * library (448 KiB on every GPU the library runs on, held until the process ends) instead of
 * cached allocations, and are rewritten by every call.  It calls no hipMalloc, hipFree or other
 * allocating routine and records no memset or copy.
 *   limit    at most 4096 non-empty tensors per call (and device numbers below 64): beyond that
 *            it returns TOA_ELIMIT and launches nothing.
 *   sharing  every call on a GPU uses that GPU's one array: calls that overlap in time on one
 *            GPU (different streams, or replays of graphs that captured it) race; calls ordered
 *            by one stream, or otherwise serialised, are safe. */
TOA_API int toa_adam_forward_inplace_multi_noalloc(int dtype, size_t num_tensors,
                                                   void *const *updates, void *const *mu,
                                                   void *const *nu, const size_t *n, double b1,
                                                   double b2, double eps, double eps_root,
                                                   const uint64_t *counts, uint64_t count_all,
                                                   void *stream);

TOA_API int toa_adam_forward_mu_multi(int dtype, size_t num_tensors, const void *const *updates,
                              const void *const *mu, const size_t *n, double b1,
                              void *const *mu_out, void *stream);

TOA_API int toa_adam_forward_nu_multi(int dtype, size_t num_tensors, const void *const *updates,
                              const void *const *nu, const size_t *n, double b2,
                              void *const *nu_out, void *stream);

TOA_API int toa_adam_forward_updates_multi(int dtype, size_t num_tensors, const void *const *new_mu,
                                   const void *const *new_nu, const size_t *n, double b1,
                                   double b2, double eps, double eps_root,
                                   const uint64_t *counts, uint64_t count_all,
                                   void *const *updates_out, void *stream);

TOA_API int toa_adam_backward_mu_multi(int dtype, size_t num_tensors, const void *const *dmu,
                               const size_t *n, double b1, void *const *dupdates_out,
                               void *const *dmu_out, void *stream);

TOA_API int toa_adam_backward_nu_multi(int dtype, size_t num_tensors, const void *const *dnu,
                               const void *const *updates, const size_t *n, double b2,
                               void *const *dupdates_out, void *const *dnu_out, void *stream);

TOA_API int toa_adam_backward_updates_multi(int dtype, size_t num_tensors, const void *const *dupdates,
                                    const void *const *updates, const void *const *new_mu,
                                    const size_t *n, double b1, double b2, double eps_root,
                                    const uint64_t *counts, uint64_t count_all,
                                    void *const *dnew_mu_out, void *const *dnew_nu_out,
                                    void *stream);

/* ---- whole differentiable step in two passes ----------------------------------
 * The differentiable branch of the reference runs three forward ops and three
 * backward ops per leaf (/root/reference/torchopt/accelerated_op/adam_op.py:167-180
 * and :52-60, :78-86, :104-121).  These entry points do each direction in one pass
 * with results bit-identical to the separate ops:
 *   forward_all   new_mu, new_nu, new_updates from one read of updates, mu, nu
 *                 (= forward_mu, forward_nu, forward_updates; 24 instead of 36 bytes
 *                 per float32 element);
 *   backward_all  d(updates), d(mu), d(nu) from d(new_updates) and the saved
 *                 new_updates, new_mu, updates (= backward_updates, then
 *                 backward_mu and backward_nu, with the additions autograd performs
 *                 between them).  dnew_mu / dnew_nu are the gradients reaching
 *                 new_mu / new_nu from outside the step; either may be NULL (for
 *                 the list form: the whole list pointer NULL), meaning none.
 * No single counterpart in the reference. */
TOA_API int toa_adam_forward_all(int dtype, const void *updates, const void *mu, const void *nu,
                                 size_t n, double b1, double b2, double eps, double eps_root,
                                 uint64_t count, void *new_mu, void *new_nu, void *new_updates,
                                 void *stream);

TOA_API int toa_adam_forward_all_multi(int dtype, size_t num_tensors,
                                       const void *const *updates, const void *const *mu,
                                       const void *const *nu, const size_t *n, double b1,
                                       double b2, double eps, double eps_root,
                                       const uint64_t *counts, uint64_t count_all,
                                       void *const *new_mu, void *const *new_nu,
                                       void *const *new_updates, void *stream);

TOA_API int toa_adam_backward_all(int dtype, const void *dnew_updates, const void *new_updates,
                                  const void *new_mu, const void *updates, const void *dnew_mu,
                                  const void *dnew_nu, size_t n, double b1, double b2,
                                  double eps_root, uint64_t count, void *dupdates, void *dmu,
                                  void *dnu, void *stream);

TOA_API int toa_adam_backward_all_multi(int dtype, size_t num_tensors,
                                        const void *const *dnew_updates,
                                        const void *const *new_updates,
                                        const void *const *new_mu, const void *const *updates,
                                        const void *const *dnew_mu, const void *const *dnew_nu,
                                        const size_t *n, double b1, double b2, double eps_root,
                                        const uint64_t *counts, uint64_t count_all,
                                        void *const *dupdates, void *const *dmu,
                                        void *const *dnu, void *stream);

/* ---- fused optimizer step ------------------------------------------------
 * The classic in-place step of `Adam(..., use_accelerated_op=True).step()` (or AdamW) in one
 * pass over memory: the Adam update (as toa_adam_forward_inplace) together with its neighbours
 * in the reference chain (paths under /root/reference/torchopt):
 *   maximize != 0               gradients are negated first (alias/utils.py:148);
 *   weight_decay, decoupled = 0 g += wd * p before the moments, as `adam` does
 *                               (alias/utils.py:113-122);
 *   weight_decay, decoupled = 1 u += wd * p after the Adam scaling, as `adamw` does
 *                               (transform/add_decayed_weights.py:232-239);
 *   updates *= -lr              (transform/scale.py:93-98 via alias/utils.py:226);
 *   params += updates           (update.py:71-74).
 * Every operation is rounded as the separate passes round it -- the two "+= wd * p" are
 * single-rounding fused multiply-adds, which is what Tensor.add_(p, alpha=wd) computes -- so
 * the result is bit-identical to them.  mu, nu and params are overwritten; `updates` is
 * overwritten with the scaled update only if write_updates != 0 (otherwise it is read only:
 * 28 instead of 32 bytes per float32 element, against 44 and more for the separate passes).
 * Element types: all four without weight decay.  On TOA_F16 / TOA_BF16 the step is forward_ with
 * the 16-bit types' per-operation rounding, then the two torch calls as torch evaluates them on
 * 16-bit tensors: the update times float(-lr) (the scalar is NOT rounded to 16 bits) rounded to
 * 16 bits, then params plus that, rounded to 16 bits.  With weight_decay != 0 the 16-bit types
 * return TOA_EDTYPE: Tensor.add_(p, alpha=wd) on 16-bit CPU tensors is not one arithmetic (its
 * vectorized body and its scalar tails round differently), so there is no result to be identical
 * to.  No single counterpart in the reference. */
TOA_API int toa_adam_fused_step(int dtype, void *params, void *updates, void *mu, void *nu,
                                size_t n, double b1, double b2, double eps, double eps_root,
                                uint64_t count, double lr, double weight_decay, int decoupled,
                                int maximize, int write_updates, void *stream);

TOA_API int toa_adam_fused_step_multi(int dtype, size_t num_tensors, void *const *params,
                                      void *const *updates, void *const *mu, void *const *nu,
                                      const size_t *n, double b1, double b2, double eps,
                                      double eps_root, const uint64_t *counts,
                                      uint64_t count_all, double lr, double weight_decay,
                                      int decoupled, int maximize, int write_updates,
                                      void *stream);

/* ---- step number on the device ----------------------------------------------
 * The reference keeps `count` as a 0-dim int64 tensor on the parameters' device
 * (/root/reference/torchopt/transform/scale_by_adam.py:401-414) and converts it to size_t on every
 * call (adam_op.cpp:32-48 through pybind11), which reads it back to the host.  The entry points
 * above take the step number as a host integer for that reason -- and a captured HIP graph then
 * replays one particular step.  The *_devcount entry points read it from device memory when the
 * kernel starts, so ONE captured graph serves a whole training loop: the graph advances the
 * count (toa_adam_count_advance, or any kernel of the caller's) and every replay computes the
 * next step.
 *
 * The bias corrections 1/(1-b1^count), 1/(1-b2^count), 1-b1^count, 1/(1-b2^count+eps_root) must
 * stay the host's (double precision with libm's pow, rounded once to the element type: that is
 * what makes results bit-identical to the reference), so the host tabulates them:
 *   toa_adam_bias_rows         fills host memory with `rows` rows of 4 values of the element type
 *                              for step numbers first_count, first_count + 1, ...; the caller
 *                              uploads them (4 * rows * element size bytes).
 *   toa_adam_bias_rows_needed  how many rows from first_count on make the table exact for EVERY
 *                              later step: the corrections stop changing once b^count is below
 *                              half an ulp of 1 (37 411 steps for b2 = 0.999).  0 if that takes
 *                              more than `limit` rows.
 *   toa_adam_count_advance     *count += (*count != INT64_MAX), the reference's inc_count
 *                              (transform/utils.py:111-126), as a one-thread kernel on `stream`.
 * A step number below first_count uses row 0, one beyond the table the last row.  `bias_rows`
 * and `count` are device pointers; `count` is read once per wavefront, when the kernel starts.
 * Entry points exist for the in-place step and the fused optimizer step, single and list (the
 * ops a training loop captures); everything else about them is as for their host-count forms.
 * No counterpart in the reference. */
TOA_API int toa_adam_bias_rows(int dtype, double b1, double b2, double eps_root,
                               uint64_t first_count, size_t rows, void *host_out);
TOA_API size_t toa_adam_bias_rows_needed(double b1, double b2, uint64_t first_count,
                                         size_t limit);
TOA_API int toa_adam_count_advance(int64_t *count, void *stream);

TOA_API int toa_adam_forward_inplace_devcount(int dtype, void *updates, void *mu, void *nu,
                                              size_t n, double b1, double b2, double eps,
                                              double eps_root, const void *bias_rows,
                                              uint64_t first_count, size_t rows,
                                              const int64_t *count, void *stream);

TOA_API int toa_adam_forward_inplace_multi_devcount(int dtype, size_t num_tensors,
                                                    void *const *updates, void *const *mu,
                                                    void *const *nu, const size_t *n, double b1,
                                                    double b2, double eps, double eps_root,
                                                    const void *bias_rows, uint64_t first_count,
                                                    size_t rows, const int64_t *count,
                                                    void *stream);

TOA_API int toa_adam_fused_step_devcount(int dtype, void *params, void *updates, void *mu,
                                         void *nu, size_t n, double b1, double b2, double eps,
                                         double eps_root, const void *bias_rows,
                                         uint64_t first_count, size_t rows, const int64_t *count,
                                         double lr, double weight_decay, int decoupled,
                                         int maximize, int write_updates, void *stream);

TOA_API int toa_adam_fused_step_multi_devcount(int dtype, size_t num_tensors, void *const *params,
                                               void *const *updates, void *const *mu,
                                               void *const *nu, const size_t *n, double b1,
                                               double b2, double eps, double eps_root,
                                               const void *bias_rows, uint64_t first_count,
                                               size_t rows, const int64_t *count, double lr,
                                               double weight_decay, int decoupled, int maximize,
                                               int write_updates, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TOA_ADAM_H */
