/*
 * nce_hip.h - C-ABI of the MI355X (gfx950) executor for the quantized NCE/DPU op path.
 *
 * The boundary is the reference's task DESCRIPTOR: one nce_cluster_task_desc_t carries what a
 * VPUIP.NCEClusterTask op carries (operands, attributes, DPUTask variants, PPETask), so a task
 * built for the NPU can be executed unchanged on the GPU.
 *
 *   descriptor operands/attrs : src/vpux_compiler/tblgen/vpux/compiler/dialect/VPUIP/ops.td:2783-2831
 *   variants (DPUTask)        : ops.td:2592-2652
 *   epilogue (PPETask)        : ops.td:2658-2743, tblgen/.../VPU/attributes.td:311-326
 *   handle / result / log style: src/vpux_driver_compiler/include/vpux_driver_compiler.h:52-68,91-100,184-185,260
 *
 * All signatures use plain pointers and sizes only. Tensor memory is caller-owned DEVICE memory
 * (hipMalloc / torch); the library never allocates or frees tensors. C++ exceptions never cross.
 */
#ifndef NCE_HIP_H
#define NCE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NCE_HIP_VERSION_MAJOR 0
#define NCE_HIP_VERSION_MINOR 1

typedef struct nce_executor_s* nce_executor_handle_t;
typedef struct nce_log_s* nce_log_handle_t;
typedef struct nce_task_list_s* nce_task_list_handle_t;

/* Same numbering as vcl_result_t (vpux_driver_compiler.h:91-100). */
typedef enum nce_result_t {
    NCE_RESULT_SUCCESS = 0,
    NCE_RESULT_ERROR_OUT_OF_MEMORY = 0x70000002,
    NCE_RESULT_ERROR_INVALID_ARGUMENT = 0x78000004,
    NCE_RESULT_ERROR_INVALID_NULL_HANDLE = 0x78000005,
    NCE_RESULT_ERROR_UNSUPPORTED = 0x78000008,
    NCE_RESULT_ERROR_IO = 0x78000009,
    NCE_RESULT_ERROR_UNKNOWN = 0x7ffffffe
} nce_result_t;

/* = VPUIP::NCETaskType (tblgen/.../VPUIP/attributes.td:80-94). FCL/IDENTITY/CMCONV: UNSUPPORTED. */
typedef enum nce_task_type_t {
    NCE_TASK_CONV = 0,
    NCE_TASK_DWCONV = 1,
    NCE_TASK_MAXPOOL = 2,
    NCE_TASK_AVEPOOL = 3,
    NCE_TASK_ELTWISE = 5
} nce_task_type_t;

/* = VPU::PPEMode values that the INT8 path uses (tblgen/.../VPU/attributes.td:263-303). */
typedef enum nce_ppe_mode_t {
    NCE_PPE_NOOP = 3,
    NCE_PPE_ADD = 5,
    NCE_PPE_LRELU = 13,
    NCE_PPE_LRELUX = 14,
    NCE_PPE_LPRELU = 15
} nce_ppe_mode_t;

/* = VPU::MPEMode (attributes.td:240-256). Carried for contract fidelity; no effect on the GPU. */
typedef enum nce_mpe_mode_t {
    NCE_MPE_VECTOR = 0,
    NCE_MPE_MATRIX = 1,
    NCE_MPE_VECTOR_FP16 = 2,
    NCE_MPE_CUBOID_16x16 = 3,
    NCE_MPE_CUBOID_8x16 = 4,
    NCE_MPE_CUBOID_4x16 = 5,
    NCE_MPE_NOP = 6
} nce_mpe_mode_t;

/* F16 / BF16 name float outputs for the parameter generators (nce_params.h) only: tasks with such tensors are rejected. */
typedef enum nce_dtype_t { NCE_DT_U8 = 0, NCE_DT_I8 = 1, NCE_DT_SI32 = 2, NCE_DT_F16 = 3, NCE_DT_BF16 = 4 } nce_dtype_t;

/* Rounding of the fixed-point right shift in the PPE (requantize and PReLU steps).
 * HALF_UP : (p + 2^(s-1)) >> s, ties toward +inf (default).  HALF_EVEN: ties to even.  NONE: floor. */
typedef enum nce_round_mode_t { NCE_ROUND_HALF_UP = 0, NCE_ROUND_HALF_EVEN = 1, NCE_ROUND_NONE = 2 } nce_round_mode_t;

/* Domain of clamp_low/clamp_high. POST_ZP: storage domain, applied after the output zero point is
 * added (37XX after SetupPPE, src/vpux_compiler/src/dialect/VPU/transforms/passes/setup_ppe.cpp:176-195).
 * PRE_ZP: zero-point-free domain, applied before it (hwtest dw/pool/eltwise builders,
 * src/vpux_translate_utils/src/hwtest/buildDWConv.cpp:264-270). */
typedef enum nce_clamp_domain_t { NCE_CLAMP_POST_ZP = 0, NCE_CLAMP_PRE_ZP = 1 } nce_clamp_domain_t;

/* A tensor operand. dims are LOGICAL [N, C, H, W] (conv weights [OC, IC, KY, KX]; depthwise weights
 * [C, pad16(KY*KX), 1, 1]; weight table [OC, 1, 1, 4]). Memory order is the one the verifier demands
 * (src/vpux_compiler/src/dialect/VPUIP/ops/nce_cluster_task.cpp:346-359,418-433,702-709): NHWC for
 * activations and OYXI for conv weights, i.e. the C / IC dimension is innermost and must be compact
 * (strides_bytes[1] == element size). The other strides are free, which is how parent_input /
 * parent_output sub-views are expressed. The OUTPUT of a task may instead use any non-overlapping strides,
 * channel stride included: that is how the ODU permutations (output written as NWHC, NWCH, NCWH, NHCW or NCHW,
 * getODUPermutationType, nce_cluster_task.cpp:764-780) are expressed; such outputs are written byte by byte. */
typedef struct nce_tensor_t {
    void* data;
    int32_t dtype;      /* nce_dtype_t */
    int32_t zero_point; /* quantization zero point of the storage type */
    int64_t dims[4];
    int64_t strides_bytes[4];
} nce_tensor_t;

/* One DPUTask variant: an output sub-box, ends INCLUSIVE, order [x, y, z] = [W, H, C]
 * (ops.td:2592-2652; nce_cluster_task.cpp:272-297). pad_* is the part of the kernel padding that
 * touches this sub-box (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/
 * runtime_dpu_parser_imports.cpp.inc:2165-2179). */
typedef struct nce_dpu_task_t {
    int32_t out_start[3];
    int32_t out_end[3];
    int32_t pad_left, pad_right, pad_top, pad_bottom;
    int32_t mpe_mode; /* nce_mpe_mode_t */
    int32_t cluster_id;
} nce_dpu_task_t;

/* The PPETask attributes (ops.td:2658-2743). Defaults of the reference: clamp = int32 min/max,
 * lrelu_mult 1, lrelu_shift 0 (ops.td:2685-2689). */
typedef struct nce_ppe_task_t {
    int32_t mode; /* nce_ppe_mode_t */
    int32_t clamp_low, clamp_high;
    int32_t lrelu_mult, lrelu_shift;
    int32_t has_quant;  /* quant_mult/quant_shift present (ELTWISE / AVEPOOL without weight table) */
    int32_t quant_mult, quant_shift, quant_post_shift;
    int32_t has_in_mult; /* in1/in2_quant_mult present (ELTWISE, 37XX per-input scales) */
    int32_t in1_quant_mult, in2_quant_mult;
    int32_t round_mode;   /* nce_round_mode_t */
    int32_t clamp_domain; /* nce_clamp_domain_t */
} nce_ppe_task_t;

/* Bits of nce_cluster_task_desc_t::flags = the boolean attributes of NCEClusterTask
 * (ops.td:2803-2817). NCE_FLAG_IS_INPLACE is accepted on ELTWISE tasks whose output IS one of the two inputs (the same
 * address, strides and storage type: what convert_eltwise_to_in_place.cpp:114-200 produces); on any other task or with
 * any other output it is NCE_RESULT_ERROR_INVALID_ARGUMENT. The other attributes are not implemented: a set bit ->
 * NCE_RESULT_ERROR_UNSUPPORTED. */
#define NCE_FLAG_IS_CONTINUED (1u << 0)
#define NCE_FLAG_IS_SEGMENTED (1u << 1)
#define NCE_FLAG_INPUT_CHANNELS_COMPRESSION (1u << 2)
#define NCE_FLAG_IS_SUPERDENSE (1u << 3)
#define NCE_FLAG_IS_INPLACE (1u << 4)
#define NCE_FLAG_IS_PERMUTE_QUANTIZE (1u << 5)
#define NCE_FLAG_IS_SMALL_KERNEL_OPTIMIZED (1u << 6)

typedef struct nce_cluster_task_desc_t {
    int32_t task_type; /* nce_task_type_t */
    uint32_t flags;
    nce_tensor_t input;
    nce_tensor_t weights;      /* CONV/DWCONV: weights. ELTWISE: second input. Pools: data == NULL. */
    nce_tensor_t weight_table; /* CONV/DWCONV: required. Pools/ELTWISE: optional (data == NULL if absent). */
    nce_tensor_t output;
    int32_t kernel_size[2];    /* [KY, KX] */
    int32_t kernel_strides[2]; /* [SY, SX] */
    int32_t kernel_pad_left, kernel_pad_right, kernel_pad_top, kernel_pad_bottom;
    const nce_dpu_task_t* variants;
    uint32_t num_variants; /* >= 1 (nce_cluster_task.cpp:588-608) */
    uint32_t reserved;
    const nce_ppe_task_t* ppe; /* NULL = NOOP with the defaults above */
} nce_cluster_task_desc_t;

typedef struct nce_executor_desc_t {
    int32_t device_id; /* HIP device ordinal; < 0: no device - the executor validates descriptors but cannot launch */
    int32_t log_level; /* 0 none, 1 error, 2 warning, 3 info, 4 debug */
} nce_executor_desc_t;

/* Library version. Style of vclGetVersion (vpux_driver_compiler.h:170-176). */
nce_result_t nceGetVersion(uint32_t* major, uint32_t* minor);

/* Create / destroy an executor bound to one GPU. Replaces the device side of
 * IEngineBackend/IDevice/Executor (src/vpux_al/include/vpux.hpp:23-117) for this op family; the
 * create(desc, out-handle, out-log) shape follows vclCompilerCreate (vpux_driver_compiler.h:184-185).
 * The log handle belongs to the executor and dies with it. Fails with ERROR_UNSUPPORTED (and a line on
 * stderr) when device_id >= 0 names no usable GPU: there is no CPU fallback. */
nce_result_t nceExecutorCreate(nce_executor_desc_t desc, nce_executor_handle_t* executor, nce_log_handle_t* log);
nce_result_t nceExecutorDestroy(nce_executor_handle_t executor);

/* Check a descriptor against the rules of NCEClusterTaskOp::verify (nce_cluster_task.cpp:610-712)
 * and verifyKernel (src/vpux_compiler/src/dialect/VPUIP/nce_invariant.cpp:1056-1108). Touches no
 * device memory. On failure the reason is appended to the log. */
nce_result_t nceClusterTaskValidate(nce_executor_handle_t executor, const nce_cluster_task_desc_t* task);

/* Validate, then launch the task on `hip_stream` (a hipStream_t; NULL = the null stream).
 * Asynchronous with respect to the host. This is what the DPU does when it consumes one task
 * descriptor (register semantics: runtime_dpu_parser_imports.cpp.inc:834-2045). */
nce_result_t nceClusterTaskEnqueue(nce_executor_handle_t executor, const nce_cluster_task_desc_t* task,
                                   void* hip_stream);

/* A recorded sequence of tasks (the GPU analogue of a VPUIP task list between two barriers
 * chains). Descriptors, variants and PPE structs are copied at Append time; tensor memory is not.
 * Enqueue launches them back to back on one stream. */
nce_result_t nceTaskListCreate(nce_executor_handle_t executor, nce_task_list_handle_t* list);
nce_result_t nceTaskListAppend(nce_task_list_handle_t list, const nce_cluster_task_desc_t* task);
nce_result_t nceTaskListEnqueue(nce_task_list_handle_t list, void* hip_stream);
/* nceTaskListEnqueue for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. It runs the list the way nceTaskListEnqueue does for an executor
 * created under NCE_HIP_PERSISTENT=1 - runs of consecutive weights-resident convolutions as one persistent launch each -
 * but keeps those launches' layer tables, counters and error word in a fixed array in device memory that belongs to the
 * library (281 KiB per GPU, held until the process ends) instead of allocating them, and calls neither hipMalloc nor
 * hipFree. (The tables travel to that array through 248 KiB of pinned host memory that every executor with a device
 * gets when it is created.) Limits: the array holds the tables of 64 layers per list - persistent launches beyond that
 * run as the ordinary launches they were made from (which allocate nothing either); a list that nceTaskListEnqueue has
 * prepared with device allocations is refused (NCE_RESULT_ERROR_INVALID_ARGUMENT); a stream that is being captured is
 * refused (NCE_RESULT_ERROR_UNSUPPORTED: every call re-stages its tables through the executor's one pinned buffer and
 * waits on an event, neither of which a graph replay would repeat - the call is eager only). Every call on a GPU shares
 * that GPU's array: calls whose launches may overlap on the GPU (two streams, two executors; two processes do not
 * share it) race and must be serialised by the caller. Failures of a persistent launch are reported by
 * nceExecutorSynchronize, as for nceTaskListEnqueue; because the array's error word and counters are shared, a failure
 * found by one executor of a GPU is reported by the next nceExecutorSynchronize of every other executor that used this
 * entry point on that GPU as well. */
nce_result_t nceTaskListEnqueueNoAlloc(nce_task_list_handle_t list, void* hip_stream);
nce_result_t nceTaskListDestroy(nce_task_list_handle_t list);

/* Wait for everything this executor enqueued on the null stream / the given stream. */
nce_result_t nceExecutorSynchronize(nce_executor_handle_t executor, void* hip_stream);

/* Two-call pattern of vclLogHandleGetString (vpux_driver_compiler.h:260): buf == NULL -> *size
 * receives the byte count including the terminator; else copies up to *size bytes and clears. */
nce_result_t nceLogHandleGetString(nce_log_handle_t log, size_t* size, char* buf);

#ifdef __cplusplus
}
#endif

#endif /* NCE_HIP_H */
