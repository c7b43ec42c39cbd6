/*
 * nce_oracle.h - CPU ORACLE for the quantized NCE/DPU op path. TEST INFRASTRUCTURE ONLY.
 *
 * This is the checker the HIP executor is compared with; nothing the library ships may call it.
 * It restates, in plain C, (1) the reference's fixed-point parameter generation and (2) the
 * per-element integer pipeline of an NCE task as the reference programs it into DPU registers.
 *
 * Pinning status (what fixes each function besides this file):
 *   - parameter generation (approximate / eltwise / prelu / table words / bias / clamps / avgpool
 *     scale): pinned by literal values held in the reference's lit tests
 *     (tests/golden/param_kats.json lists value + file:line).
 *   - per-element pipeline (nce_oracle_run, nce_oracle_ppe, nce_oracle_rshift_round):
 *     the reference holds NO executable implementation and no golden output for it (it runs in NPU
 *     hardware), so against the reference it is "parity unpinned". It is pinned here by closed
 *     forms, an independent numpy im2col/int64 formulation, torch int64 conv2d, cross-task
 *     invariants and exhaustive rounding checks (tests/test_oracle_pipeline.py).
 */
#ifndef NCE_ORACLE_H
#define NCE_ORACLE_H

#include <stdint.h>

#include "../include/nce_hip.h" /* descriptor structs only */

#ifdef __cplusplus
extern "C" {
#endif

enum { NCE_ORACLE_ARCH_30XX = 0, NCE_ORACLE_ARCH_37XX = 1 };

/* ---- parameter generation ---------------------------------------------------------------- */

/* approximate<T>(bits, target): src/vpux_compiler/src/utils/quantization.cpp:242-252 */
void nce_oracle_approximate(int bits, double target, int64_t* mult, int32_t* shift, int32_t* post_shift);

/* QuantizationApproximation (15 bit): quantization.cpp:256-264. Returns 0, or -1 when post_shift != 0
 * on an architecture that does not allow it. */
int nce_oracle_quant_approx(int arch, double target, int32_t* mult, int32_t* shift, int32_t* post_shift);

/* EltwiseQuantizationApproximation: quantization.cpp:286-330. Returns 0, or -1 when the reference
 * throws ("out of register range"). */
int nce_oracle_eltwise_approx(int arch, double in1_scale, double in2_scale, double out_scale, int32_t* in1_mult,
                              int32_t* in2_mult, int32_t* out_mult, int32_t* out_shift);

/* PReLUApproximation: quantization.cpp:344-354 (11 bit on 37XX, 7 bit on 30XX). */
int nce_oracle_prelu_approx(int arch, double alpha, int32_t* mult, int32_t* shift);

/* Weights-table word [2]: src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:122-155.
 * lrelu_mult >= 0 applies the 30XX LPRELU low-byte overwrite (:227-232); pass -1 otherwise. */
int32_t nce_oracle_scale_word(int arch, int32_t shift, int32_t mult, int32_t lrelu_mult);

/* IEEE-754 bits of (float)x: toHex, nce_sparsity.cpp:31-33 (37XX float-input table words). */
int32_t nce_oracle_float_bits(double x);

/* Weights-table word [3] for quantized input: round(bias / (w_scale*in_scale)), half away from
 * zero (nce_sparsity.cpp:186-193, 646-676). Returns -1 if the value leaves int32. */
int nce_oracle_rescaled_bias(double bias_fp, double w_scale, double in_scale, int32_t* out);

/* getWeightsTable for quantized in/out on 37XX/30XX: nce_sparsity.cpp:445-519. table is OC x 4 int32.
 * w_scales has n_w_scales (1 or OC) entries; bias_fp may be NULL. Returns 0 / -1. */
int nce_oracle_weights_table(int arch, int32_t oc, int32_t weight_ptr_base, int32_t weight_ptr_step,
                             int32_t sparsity_ptr, double in_scale, double out_scale, const double* w_scales,
                             int32_t n_w_scales, const double* bias_fp, int32_t lrelu_mult, int32_t* table);

/* calculateQuantScaleVectorForAvgPool, quantized in/out: src/vpux_compiler/src/utils/VPU/ppe_utils.cpp:72-106 */
double nce_oracle_avgpool_scale(double in_scale, double out_scale, int32_t ky, int32_t kx);

/* Post-ops understood by parsePostOp (ppe_utils.cpp:293-376). */
enum { NCE_ORACLE_POSTOP_NONE = 0, NCE_ORACLE_POSTOP_RELU = 1, NCE_ORACLE_POSTOP_CLAMP = 2, NCE_ORACLE_POSTOP_LEAKY_RELU = 3 };

/* Stage 1 (IE -> VPU.NCE): PPE attributes for a quantized output, zero-point-free clamp domain
 * (ppe_utils.cpp:293-376, quantization.cpp:364-380; no post-op: ppe_utils.cpp:151-156).
 * Fills mode, clamp_low, clamp_high, lrelu_mult, lrelu_shift; sets clamp_domain = PRE_ZP.
 * a0 = alpha (LEAKY_RELU) or clamp min (CLAMP); a1 = clamp max. Returns 0 / -1. */
int nce_oracle_ppe_stage1(int arch, int postop, double a0, double a1, int32_t storage_min, int32_t storage_max,
                          double out_scale, int32_t out_zp, nce_ppe_task_t* ppe);

/* Stage 2 (37XX SetupPPE): rewrite to storage-domain clamps and recompute the mode
 * (src/vpux_compiler/src/dialect/VPU/transforms/passes/setup_ppe.cpp:12-33,123-195).
 * has_ppe = 0 models an op that had no PPE attribute at all. Sets clamp_domain = POST_ZP. */
void nce_oracle_ppe_stage2_37xx(int has_ppe, int32_t storage_min, int32_t storage_max, int32_t out_zp,
                                nce_ppe_task_t* ppe);

/* FuseClamp for a quantized (per-tensor) output: ClampConverter::getTargetClamps,
 * src/vpux_compiler/src/dialect/VPU/transforms/passes/fuse_clamp.cpp:34-53. Rewrites *clamp_low / *clamp_high (the
 * op's PPE range on entry). The mode does not change for quantized outputs (:74-78). Returns 0 / -1. */
int nce_oracle_fuse_clamp_quant(double out_scale, int32_t out_zp, double clamp_min, double clamp_max, int32_t* clamp_low,
                                int32_t* clamp_high);

/* ---- per-element integer pipeline ---------------------------------------------------------- */

int64_t nce_oracle_rshift_round(int64_t p, int32_t shift, int32_t round_mode);

/* Steps 1-6 of the PPE for one accumulator value: +bias, *mult >> shift, PReLU, +zp, clamp,
 * saturate to the output type. Register order: runtime_dpu_parser_imports.cpp.inc:511-542,1952-2045. */
int32_t nce_oracle_ppe(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const nce_ppe_task_t* ppe,
                       int32_t out_zp, int32_t out_dtype);

/* Evaluate one task with HOST pointers in the descriptor. Returns 0, or a negative code for a
 * descriptor it cannot evaluate. nthreads <= 0: use all cores. */
int nce_oracle_run(const nce_cluster_task_desc_t* task, int nthreads);

/* Threads nce_oracle_run uses for nthreads <= 0. */
int nce_oracle_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
