/*
 * TEST-ONLY entry points of libtrtamd_bert_plugins.so.
 *
 * Nothing in a product path calls these: the IPluginV3 classes, the encoder runner and the bindings of
 * include/trtamd_bert_kernels.h never reference them.  They exist so that the parity tests can look at values a
 * fused kernel otherwise keeps in registers.  They have no counterpart in the reference (its fused kernels are
 * precompiled binaries without such a view).
 */
#ifndef TRTAMD_TEST_HOOKS_H
#define TRTAMD_TEST_HOOKS_H

#include "trtamd_bert_kernels.h"

#ifdef __cplusplus
extern "C"
{
#endif

/* trtamd_fused_mha_run with a dump of intermediates: the same launch through the kernel instantiation that also
 * stores the first GEMM's accumulators (acc1: [b][h][s][s], int32 for INT8, binary32 bit patterns for FP16;
 * entries (query, key) beyond a sequence's length are left untouched) and, for INT8, the quantised probabilities
 * (p8: [b][h][s][s] int8).  Either pointer may be NULL.  The context output is bit-identical to
 * trtamd_fused_mha_run's, which the tests assert. */
TRTAMD_API int trtamd_fused_mha_run_debug(trtamd_stream_t stream, int32_t data_type, trtamd_fmha_params const* params,
    int32_t* acc1, int8_t* p8);

/* Tuning switches (README, "Tuning switches"): kernel variants other than the default choice.  A process normally
 * selects them with an environment variable of the same name, read once; these two calls let one test process walk
 * through the settings instead.  name: the variable's name, e.g. "TRTAMD_LINEAR_DIRECT"; value: what atoi() of the
 * variable would give.  trtamd_test_reset_tuning returns the switch to the environment's (or the default) value.
 * An unknown name returns TRTAMD_STATUS_BAD_PARAM. */
TRTAMD_API int trtamd_test_set_tuning(char const* name, int32_t value);
TRTAMD_API int trtamd_test_reset_tuning(char const* name);

#ifdef __cplusplus
}
#endif

#endif /* TRTAMD_TEST_HOOKS_H */
