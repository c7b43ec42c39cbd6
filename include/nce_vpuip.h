/*
 * nce_vpuip.h - importer for the textual form of compiler-emitted VPUIP programs: the sequence of
 * VPURT.DeclareBuffer / VPUIP.NCEClusterTask / VPUIP.NNDMA operations the reference prints after lowering
 * (e.g. tests/lit/NPU/conversion/passes/VPUIP2VPUMI37XX/nce_eltwise_37XX.mlir:18-34, nce_conv_37XX.mlir:36-47,
 * nce_maxpool_37XX.mlir:17-33; op syntax src/vpux_compiler/tblgen/vpux/compiler/dialect/VPUIP/ops.td:2749-3019,
 * printer src/vpux_compiler/src/dialect/VPUIP/ops/nce_cluster_task.cpp). It turns every NCEClusterTask into the
 * descriptor of nce_hip.h and runs the program in order on one HIP stream.
 *
 * What is read: `#NAME = affine_map<...>` and `!NAME = ...` aliases; the arguments of the (first) func.func;
 * `%n = VPURT.DeclareBuffer <SECTION> [indices] <byte offset> -> memref<...>`; NCEClusterTask with its attribute
 * dictionary, operand list, `variants : { DPUTask {...} ... }` and `PPE : { PPETask <MODE> {...} }`; and
 * `VPUIP.NNDMA ... inputs(%a : T) outputs(%b : T)` as a plain copy. Barriers, VPURT.Task wrappers, IE.CNNNetwork and
 * everything else are skipped: a single in-order stream gives the same ordering the barriers encode.
 * Memory is the caller's: each (section, index) pair - CMX_NN per cluster, DDR, the function arguments - is bound
 * to a base pointer, and a buffer's address is base + byte offset.
 */
#ifndef NCE_VPUIP_H
#define NCE_VPUIP_H

#include "nce_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nce_vpuip_program_s* nce_vpuip_program_handle_t;

typedef enum nce_vpuip_section_t {
    NCE_VPUIP_SECTION_ARGUMENT = 0, /* func.func argument number `index` (network inputs, then outputs) */
    NCE_VPUIP_SECTION_CMX_NN = 1,   /* VPURT.DeclareBuffer <CMX_NN> [cluster] */
    NCE_VPUIP_SECTION_DDR = 2,      /* VPURT.DeclareBuffer <DDR> */
    NCE_VPUIP_SECTION_NETWORK_INPUT = 3,
    NCE_VPUIP_SECTION_NETWORK_OUTPUT = 4
} nce_vpuip_section_t;

typedef enum nce_vpuip_op_kind_t { NCE_VPUIP_OP_NCE_TASK = 0, NCE_VPUIP_OP_DMA = 1 } nce_vpuip_op_kind_t;

/* A declared buffer or function argument. Element type: nce_dtype_t for u8 / i8 / si32, -1 for anything else
 * (f16, i1, ...: such buffers can be bound and copied but not used by an NCE task here). */
typedef struct nce_vpuip_buffer_t {
    char name[32];          /* SSA name, e.g. "%3" or "%arg0" */
    int32_t section, index; /* nce_vpuip_section_t, cluster / argument number */
    int64_t byte_offset;    /* inside the section */
    int64_t byte_size;      /* span the strides cover */
    int32_t dtype;
    int32_t elem_bytes;
    int32_t zero_point;
    int64_t dims[4];          /* logical N, C, H, W */
    int64_t strides_bytes[4]; /* per logical dimension */
} nce_vpuip_buffer_t;

typedef struct nce_vpuip_info_t {
    int32_t num_buffers, num_ops, num_tasks, num_dmas;
    char function[64];
} nce_vpuip_info_t;

/* Parse a program. Syntax errors and unsupported constructs INSIDE an NCEClusterTask (sparsity operands, storage
 * element tables, distributed buffer types) are reported in the log with the line number and fail the parse. */
nce_result_t nceVpuipParse(const char* mlir_text, nce_vpuip_program_handle_t* program, nce_log_handle_t log);
nce_result_t nceVpuipDestroy(nce_vpuip_program_handle_t program);
nce_result_t nceVpuipGetInfo(nce_vpuip_program_handle_t program, nce_vpuip_info_t* info);
nce_result_t nceVpuipGetBuffer(nce_vpuip_program_handle_t program, int32_t i, nce_vpuip_buffer_t* buffer);
/* Kind of operation i (program order) and, for an NCE task, its index among the tasks. */
nce_result_t nceVpuipGetOp(nce_vpuip_program_handle_t program, int32_t i, int32_t* kind, int32_t* task_index);

/* Bind the memory behind one (section, index): every buffer declared there must fit in size_bytes. */
nce_result_t nceVpuipBind(nce_vpuip_program_handle_t program, int32_t section, int32_t index, void* base, int64_t size_bytes);

/* Descriptor of NCE task number `task_index` with data pointers resolved through the bindings. The variant
 * array and PPE task it points to belong to the program and live until nceVpuipDestroy. */
nce_result_t nceVpuipGetTask(nce_vpuip_program_handle_t program, int32_t task_index, nce_cluster_task_desc_t* desc,
                             nce_log_handle_t log);

/* Run the whole program in order: NCE tasks through nceClusterTaskEnqueue, DMAs as device copies (dense,
 * equal-sized source and destination only). Asynchronous with respect to the stream. */
nce_result_t nceVpuipEnqueue(nce_vpuip_program_handle_t program, nce_executor_handle_t executor, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* NCE_VPUIP_H */
