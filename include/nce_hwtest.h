/*
 * nce_hwtest.h - front end for the reference's single-operation hardware test descriptors
 * ("config.json" of the PSS / hwtest flow): parse the JSON text, then fill an NCE task descriptor, its
 * DPU variant, PPE attributes and weights table the way the reference's test builders do, so that those
 * descriptors run unchanged on the GPU executor of nce_hip.h.
 *
 * Replaces, for the five NCE task types:
 *   parser   : nb::TestCaseJsonDescriptor, src/vpux_translate_utils/src/hwtest/test_case_json_parser.cpp:386-407
 *              (quantization), :464-585 (input / weight / output), :640-742 (conv_op / pool_op), :744-790
 *              (activation), :847-1026 (top level, per case type)
 *   builders : src/vpux_translate_utils/src/hwtest/buildZMConvTest.cpp:56-423, buildDWConv.cpp:50-302,
 *              buildMaxPoolTest.cpp, buildAvgPoolTest.cpp:30-215, buildEltwiseTest.cpp:20-204
 * Everything else in that flow (buffer placement in CMX, DMA tasks, barriers, blob emission) has no GPU
 * counterpart: the caller owns the device buffers and enqueues the filled descriptor.
 */
#ifndef NCE_HWTEST_H
#define NCE_HWTEST_H

#include "nce_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nce_hwtest_case_s* nce_hwtest_case_handle_t;

/* nb::ActivationType (test_case_json_parser.hpp:212-224). */
typedef enum nce_hwtest_activation_t {
    NCE_HWTEST_ACT_NONE = 0,
    NCE_HWTEST_ACT_RELU = 1,
    NCE_HWTEST_ACT_RELUX = 2,
    NCE_HWTEST_ACT_LEAKY_RELU = 3, /* "LeakyReLU" or "PReLU" */
    NCE_HWTEST_ACT_OTHER = 4       /* Mish, HSwish, Sigmoid, ...: parsed, not executable here */
} nce_hwtest_activation_t;

#define NCE_HWTEST_MAX_SCALES 4096

/* One "input" / "weight" / "output" entry (nb::InputLayer / WeightLayer / OutputLayer + nb::QuantParams). */
typedef struct nce_hwtest_layer_t {
    int32_t present;
    int32_t dtype;        /* nce_dtype_t, or -1 for a type this executor does not run (fp16, int4, ...) */
    char dtype_name[16];  /* as written in the JSON, e.g. "uint8" */
    int64_t shape[4];     /* logical N, C, H, W (weights: OC, IC, KY, KX) */
    int32_t has_quant;
    int32_t num_scales;   /* 1 = per tensor, OC = per channel */
    double scale0;        /* first scale; all of them through nceHwtestGetScales */
    int64_t zero_point, low_range, high_range;
    char file_path[256];  /* weights only ("file_path"), may be empty */
} nce_hwtest_layer_t;

typedef struct nce_hwtest_case_t {
    int32_t arch;              /* nce_arch_t of nce_params.h: 0 = VPUX30XX, 1 = VPUX37XX */
    char case_type[48];        /* as written, e.g. "ZMajorConvolution" */
    int32_t task_type;         /* nce_task_type_t this case maps to, or -1 (DMA, ActShave, sparse cases, ...) */
    nce_hwtest_layer_t input;  /* first entry of "input" */
    nce_hwtest_layer_t weight; /* first entry of "weight" (EltwiseDense: the second operand) */
    nce_hwtest_layer_t output; /* first entry of "output" */
    int32_t kernel[2];         /* [KY, KX]: weight shape (conv) or pool_op.kernel_shape */
    int32_t stride[2];         /* [SY, SX] */
    int32_t pad[4];            /* as written: [top, left, bottom, right] (hwtest_utils.hpp:24-35) */
    int32_t group, dilation;
    int32_t compress, act_sparsity;
    int32_t mpe_mode;          /* nce_mpe_mode_t (conv_op.mpe_mode; default CUBOID_16x16) */
    int32_t activation;        /* nce_hwtest_activation_t */
    double alpha, maximum;
    char output_order[8];      /* "nhwc" unless an ODU permutation is requested */
    char ew_mode[8];           /* "ADD" / "SUB" / "MULT" */
} nce_hwtest_case_t;

/* Parse a descriptor. Lines that start with "//" are dropped first, as the reference does for LIT inputs
 * (test_case_json_parser.cpp:22-36). Errors carry the reference's messages ("Failed to get architecture",
 * "loadConvLayer: missing strides", ...) in the log and return NCE_RESULT_ERROR_INVALID_ARGUMENT. `log` may be
 * NULL. */
nce_result_t nceHwtestParse(const char* json_text, nce_hwtest_case_handle_t* out_case, nce_log_handle_t log);
nce_result_t nceHwtestDestroy(nce_hwtest_case_handle_t hw_case);
nce_result_t nceHwtestGetCase(nce_hwtest_case_handle_t hw_case, nce_hwtest_case_t* out);
/* which: 0 input, 1 weight, 2 output. Copies min(capacity, num_scales) scales. */
nce_result_t nceHwtestGetScales(nce_hwtest_case_handle_t hw_case, int32_t which, double* scales, int32_t capacity);

/* Fill a task the way the case's builder does. On return `desc` holds task type, dtypes, zero points, logical
 * dims and DENSE strides (inputs NHWC, weights OYXI, output in the case's output_order; data pointers NULL: the
 * caller sets them), kernel / stride / pad, one
 * whole-output variant in `variant` and the PPE attributes in `ppe` (desc->variants / desc->ppe point at them).
 * `table` receives OC rows of 4 int32 when the builder emits a weights table (CONV, DWCONV; pools / eltwise only
 * for per-channel output scales); *table_rows tells how many rows were written (0 = no table).
 * Depthwise weights are described in their padded memory form [C, 16 * ceil(KY*KX / 16)].
 * A ZMajorConvolution whose input channels are no multiple of 16 is described over PADDED buffers, as its builder
 * allocates them (buildZMConvTest.cpp:111-136): desc->input.dims[1] and desc->weights.dims[1] are the channel count
 * rounded up to 16; the caller supplies weights whose padding channels hold the weights' zero point (any bytes may
 * sit in the padding channels of the input).
 * Returns NCE_RESULT_ERROR_UNSUPPORTED for case types, data types or activations the executor cannot run (the log
 * names which). */
nce_result_t nceHwtestBuildTask(nce_hwtest_case_handle_t hw_case, nce_cluster_task_desc_t* desc, nce_dpu_task_t* variant,
                                nce_ppe_task_t* ppe, int32_t* table, int32_t table_capacity_rows, int32_t* table_rows,
                                nce_log_handle_t log);

/* Case types that the reference builds as several NCE tasks (one program per case):
 *   DoubleZMajorConvolution  two chained convolutions through a tensor of the output's type (buildDoubleConvTest.cpp:55-492)
 *   RaceConditionDPU         the same convolution on num_clusters clusters, iteration_count times each; every cluster's
 *                            output must hold the same bytes (buildRaceConditionDPUTest.cpp:41-243)
 *   DifferentClustersDPU     one convolution whose output goes to every cluster of DPUTaskParams.output_cluster
 *                            (buildDIfferentClustersDPUTest.cpp:25-260)
 *   MultiClustersDPU         one convolution split over DPUTaskParams.task_clusters along the rows (SOH) or the output
 *                            channels (SOK), each cluster one workload (buildMultiClustersDPUTest.cpp:289-626)
 * None of them adds a PPE task. A GPU has no clusters: a "cluster" is one output tensor and, for MultiClustersDPU, one
 * workload (variant) whose cluster_id names it. */
#define NCE_HWTEST_MAX_OUTPUTS 8

typedef struct nce_hwtest_program_t {
    int32_t num_tasks;          /* tasks to run, in order, on one stream (what the program's barriers encode) */
    int32_t num_outputs;        /* tensors the program returns: one per cluster where the case names clusters */
    int32_t num_intermediates;  /* 1 for DoubleZMajorConvolution (the first convolution's output), else 0 */
    int32_t outputs_identical;  /* 1: every output must hold the same bytes */
    int64_t output_shape[NCE_HWTEST_MAX_OUTPUTS][4]; /* logical N, C, H, W of each output (type: the case's output) */
    int64_t intermediate_shape[4];                   /* dense NHWC, the output's type and zero point */
} nce_hwtest_program_t;

/* Which tensors task `index` reads and writes. The descriptor's data pointers are NULL; the caller sets
 * input.data = base of the input tensor + input_offset_bytes, output.data = base of the output tensor +
 * output_offset_bytes, weights.data = the weights of entry weight_layer of "weight" + weights_offset_bytes. The offsets
 * are non-zero where a cluster computes a slice into a tensor of its own (MultiClustersDPU without broadcast): the task
 * is then the convolution over the input rows / the weights rows that slice needs. */
typedef struct nce_hwtest_binding_t {
    int32_t input_tensor;   /* -1: the case's input; 0: the intermediate tensor */
    int32_t output_tensor;  /* >= 0: output of that index; -1: the intermediate tensor */
    int32_t weight_layer;   /* entry of "weight" */
    int32_t reserved;
    int64_t input_offset_bytes, output_offset_bytes, weights_offset_bytes;
} nce_hwtest_binding_t;

nce_result_t nceHwtestGetProgram(nce_hwtest_case_handle_t hw_case, nce_hwtest_program_t* out, nce_log_handle_t log);
/* nceHwtestBuildTask for task `index` of the case's program (index 0 of a single-task case is that task). */
nce_result_t nceHwtestBuildTaskAt(nce_hwtest_case_handle_t hw_case, int32_t index, nce_cluster_task_desc_t* desc,
                                  nce_dpu_task_t* variant, nce_ppe_task_t* ppe, int32_t* table, int32_t table_capacity_rows,
                                  int32_t* table_rows, nce_hwtest_binding_t* binding, nce_log_handle_t log);

#ifdef __cplusplus
}
#endif
#endif /* NCE_HWTEST_H */
