/*
 * nce_params.h - fixed-point parameter generation for NCE tasks: from quantization scales, zero
 * points, bias and post-op to the weight table and the PPE task attributes a descriptor carries.
 * Host-only arithmetic (no GPU needed); it closes the step the reference performs when it lowers
 * an IE op to VPU.NCE (src/vpux_compiler/src/VPU37XX/conversion/passes/IE2VPU/convert_IE_to_VPU_NCE.cpp:28-200).
 */
#ifndef NCE_PARAMS_H
#define NCE_PARAMS_H

#include "nce_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum nce_arch_t { NCE_ARCH_VPUX30XX = 0, NCE_ARCH_VPUX37XX = 1 } nce_arch_t;

typedef enum nce_postop_t {
    NCE_POSTOP_NONE = 0,
    NCE_POSTOP_RELU = 1,      /* IE.ReLU */
    NCE_POSTOP_CLAMP = 2,     /* IE.Clamp {min, max} */
    NCE_POSTOP_LEAKY_RELU = 3 /* IE.LeakyRelu {negative_slope} */
} nce_postop_t;

/* Per-tensor quantization of an activation: real = scale * (q - zero_point). */
typedef struct nce_quant_t {
    double scale;
    int32_t zero_point;
    int32_t dtype; /* nce_dtype_t: U8 or I8 */
} nce_quant_t;

/* QuantizationApproximation: src/vpux_compiler/src/utils/quantization.cpp:242-264 (15-bit mantissa). */
nce_result_t nceQuantApproximate(int32_t arch, double target, int32_t* mult, int32_t* shift, int32_t* post_shift);

/* EltwiseQuantizationApproximation: quantization.cpp:286-330. */
nce_result_t nceEltwiseQuantApproximate(int32_t arch, double in1_scale, double in2_scale, double out_scale,
                                        int32_t* in1_mult, int32_t* in2_mult, int32_t* out_mult, int32_t* out_shift);

/* PReLUApproximation: quantization.cpp:344-354. */
nce_result_t ncePReLUApproximate(int32_t arch, double alpha, int32_t* mult, int32_t* shift);

/* NCESparsity::getWeightsTable for quantized input and output:
 * src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:445-519 (+ :141-155 word [2], :157-222 bias).
 * table receives oc rows of 4 int32 = {weights ptr, sparsity ptr, (mult<<16)|(shift<<8), bias}.
 * weight_scales has n_weight_scales (1 or oc) entries; bias may be NULL (all zero). */
nce_result_t nceWeightsTableFill(int32_t arch, int32_t oc, int32_t weights_ptr, int32_t weights_ptr_step,
                                 int32_t sparsity_ptr, double in_scale, double out_scale,
                                 const double* weight_scales, int32_t n_weight_scales, const double* bias,
                                 int32_t* table);

/* PPE attributes of a CONV / DWCONV / MAXPOOL task with a quantized output: parsePostOp
 * (src/vpux_compiler/src/utils/VPU/ppe_utils.cpp:293-376), then, for 37XX, the SetupPPE rewrite to
 * storage-domain clamps (src/vpux_compiler/src/dialect/VPU/transforms/passes/setup_ppe.cpp:12-33,123-195).
 * p0 = negative slope (LEAKY_RELU) or min (CLAMP); p1 = max (CLAMP). */
nce_result_t ncePpeFromPostOp(int32_t arch, int32_t postop, double p0, double p1, nce_quant_t out, nce_ppe_task_t* ppe);

/* getNCEAveragePoolPPETaskAttr, quantized: ppe_utils.cpp:136-184 (scale in/out/(KY*KX) in the PPE). */
nce_result_t ncePpeForAvgPool(int32_t arch, nce_quant_t in, nce_quant_t out, int32_t ky, int32_t kx, int32_t postop,
                              double p0, double p1, nce_ppe_task_t* ppe);

/* getNCEEltwisePPETaskAttr for ADD, quantized: ppe_utils.cpp:186-253 (per-input multipliers on 37XX). */
nce_result_t ncePpeForEltwiseAdd(int32_t arch, nce_quant_t in1, nce_quant_t in2, nce_quant_t out, int32_t postop,
                                 double p0, double p1, nce_ppe_task_t* ppe);

/* FuseClamp: fold a Clamp {min, max} that follows an NCE op into the op's PPE attributes -
 * ClampConverter::getTargetClamps and getPPEMode,
 * src/vpux_compiler/src/dialect/VPU/transforms/passes/fuse_clamp.cpp:34-83. ppe is read and rewritten.
 * out.dtype U8 / I8 (per-tensor quantized): clamp_low = max(clamp_low, round(min / scale) + zp), clamp_high =
 * min(clamp_high, round(max / scale) + zp), mode unchanged. out.dtype F16 / BF16: clamp_low = INT32_MIN, clamp_high =
 * min(clamp_high, bits of max in that type), mode LRELUX. Returns ERROR_UNSUPPORTED, ppe untouched, where the reference
 * keeps the Clamp as an op of its own (isLegalClamp, fuse_clamp.cpp:123-147): a float output with min != 0. */
nce_result_t ncePpeFuseClamp(nce_quant_t out, double clamp_min, double clamp_max, nce_ppe_task_t* ppe);

/* Bytes of one output channel's weight set and of the zero padding that completes it to a multiple of 16 bytes:
 * IC*KY*KX elements are flattened to [OC, 1, 1, IC*KY*KX] and padded when that count is no multiple of 16
 * (alignConvWeightsTensor, src/vpux_compiler/src/dialect/VPU/utils/const_utils.cpp:245-285; the step of the weight
 * table pointers, getWeightPtrStep, src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:388-413). */
nce_result_t nceConvWeightSetBytes(int64_t ic, int64_t ky, int64_t kx, int64_t* set_bytes, int64_t* pad_bytes);

/* Check words [0] and [1] of a HOST copy of a weight table against the contract the executor relies on: word [0] of
 * row oc equals word [0] of row 0 plus oc * weights_ptr_step, every pointer a multiple of 16
 * (nce_sparsity.cpp:504-510), word [1] the dense marker 0xFFFFFF (nce_sparsity.hpp:32). The executor itself never
 * dereferences device memory on the host, so it cannot make this check; callers that build tables do. */
nce_result_t nceWeightsTableCheck(const int32_t* table, int32_t oc, int32_t weights_ptr_step);

#ifdef __cplusplus
}
#endif
#endif /* NCE_PARAMS_H */
