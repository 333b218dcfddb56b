/*
 * Test hooks of the sampling engine. They exist only in libftk_sampling_hooks.so, a second build of
 * libftk_sampling.so compiled with -DFTK_TEST_HOOKS for the test-suite; the product library does not export
 * them and has none of the process-wide switches they set. None of them has a counterpart in the reference.
 */
#ifndef FTK_TEST_HOOKS_H
#define FTK_TEST_HOOKS_H

#include "ftk_sampling.h"

#ifdef __cplusplus
extern "C" {
#endif

/* host-side instances of the arithmetic shared by all kernels */
float ftk_host_expf(float x);
float ftk_host_logf(float x);
/* raw Philox-4x32-10 block for known-answer tests (host) */
void ftk_host_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
/* kind 0: det_expf, 1: det_logf, 2: float->half->float, 3: float->bf16->float, 4: 1/(x+1e-6), 5: subnormal
 * arithmetic, 6: det_expf_nonpos (x <= 0 or NaN), 7: `in` holds (numerator, denominator) pairs, out[2j] = the
 * quotient by the shared-reciprocal sequence of the softmax, out[2j+1] = the ordinary division; n elements on
 * device */
int ftk_test_device_math(int kind, const float* in, float* out, size_t n, ftk_stream_t stream);
/* draws `n_draws` uniforms per row into out[row*n_draws + i], advancing the states */
int ftk_test_rng_uniform(ftk_rng_state* states, float* out, int batch_size, int n_draws, ftk_stream_t stream);
/* non-zero: every top-p row takes the radix-sort fallback (exercises it on small inputs); process-wide */
void ftk_test_set_topp_force_deep(int enable);
/* non-zero: every fused step takes the general stream, also where the lean gather would run; process-wide */
void ftk_test_set_fused_force_general(int enable);
/* non-zero: the fused step keeps gather and selection in two launches also where one workgroup per row could do
   both in one; process-wide */
void ftk_test_set_fused_two_launches(int enable);
/* which kernels the last fused step of this process launched: 0 general stream, 1 lean gather + select, 2 lean gather
   that also selects (one 256-thread workgroup per row), 3 one 1024-thread workgroup per row, 4 log-prob step, 5 large-k lists in one launch + select;
   -1 before the first step */
int ftk_test_last_fused_path(void);
/* the form of the fused log-prob step: 0 the product's choice, 1 two launches (row maxima, then one 256-thread
   workgroup per row), 1024 / 512 / 256 one launch with that many threads per row; process-wide */
void ftk_test_set_lp_form(int form);
/* non-zero keeps launches with a large k (beyond 192) on the two launches of the lean gather also where one
   1024-thread workgroup per row would make the rows' lists in one launch; process-wide */
void ftk_test_set_largek_two_launches(int on);
/* the beam-search step: 1 = sections of rows in three launches everywhere, 2 = one 1024-thread workgroup per row in
   one launch everywhere, 3 = the same with 512 threads, 0 = chosen by the shape (the product's behaviour);
   process-wide */
void ftk_test_set_beam_path(int path);

#ifdef __cplusplus
}
#endif
#endif /* FTK_TEST_HOOKS_H */
