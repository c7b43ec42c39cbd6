"""ctypes view of include/nce_hip.h, nce_params.h, nce_hwtest.h and nce_vpuip.h, and the loader of libnce_hip.so.

The shared library is the product: loading fails loudly when it has not been built, and nothing
here falls back to a CPU implementation.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# NCE_HIP_LIB points the loader at another build of the same library (kernel experiments).
LIB_PATH = os.environ.get("NCE_HIP_LIB") or os.path.join(_HERE, "libnce_hip.so")

# nce_result_t
SUCCESS = 0
ERROR_OUT_OF_MEMORY = 0x70000002
ERROR_INVALID_ARGUMENT = 0x78000004
ERROR_INVALID_NULL_HANDLE = 0x78000005
ERROR_UNSUPPORTED = 0x78000008
ERROR_IO = 0x78000009
ERROR_UNKNOWN = 0x7FFFFFFE
RESULT_NAMES = {
    SUCCESS: "NCE_RESULT_SUCCESS",
    ERROR_OUT_OF_MEMORY: "NCE_RESULT_ERROR_OUT_OF_MEMORY",
    ERROR_INVALID_ARGUMENT: "NCE_RESULT_ERROR_INVALID_ARGUMENT",
    ERROR_INVALID_NULL_HANDLE: "NCE_RESULT_ERROR_INVALID_NULL_HANDLE",
    ERROR_UNSUPPORTED: "NCE_RESULT_ERROR_UNSUPPORTED",
    ERROR_IO: "NCE_RESULT_ERROR_IO",
    ERROR_UNKNOWN: "NCE_RESULT_ERROR_UNKNOWN",
}

# nce_task_type_t = VPUIP::NCETaskType
TASK_CONV, TASK_DWCONV, TASK_MAXPOOL, TASK_AVEPOOL, TASK_ELTWISE = 0, 1, 2, 3, 5
# nce_ppe_mode_t = VPU::PPEMode
PPE_NOOP, PPE_ADD, PPE_LRELU, PPE_LRELUX, PPE_LPRELU = 3, 5, 13, 14, 15
# nce_mpe_mode_t = VPU::MPEMode
MPE_VECTOR, MPE_MATRIX, MPE_VECTOR_FP16, MPE_CUBOID_16x16, MPE_CUBOID_8x16, MPE_CUBOID_4x16, MPE_NOP = range(7)
# nce_dtype_t
DT_U8, DT_I8, DT_SI32, DT_F16, DT_BF16 = 0, 1, 2, 3, 4
# nce_round_mode_t / nce_clamp_domain_t
ROUND_HALF_UP, ROUND_HALF_EVEN, ROUND_NONE = 0, 1, 2
CLAMP_POST_ZP, CLAMP_PRE_ZP = 0, 1
# nce_arch_t / nce_postop_t (nce_params.h)
ARCH_VPUX30XX, ARCH_VPUX37XX = 0, 1
POSTOP_NONE, POSTOP_RELU, POSTOP_CLAMP, POSTOP_LEAKY_RELU = 0, 1, 2, 3

INT32_MIN, INT32_MAX = -(2**31), 2**31 - 1


class Tensor(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("dtype", C.c_int32),
        ("zero_point", C.c_int32),
        ("dims", C.c_int64 * 4),
        ("strides_bytes", C.c_int64 * 4),
    ]


class DpuTask(C.Structure):
    _fields_ = [
        ("out_start", C.c_int32 * 3),
        ("out_end", C.c_int32 * 3),
        ("pad_left", C.c_int32),
        ("pad_right", C.c_int32),
        ("pad_top", C.c_int32),
        ("pad_bottom", C.c_int32),
        ("mpe_mode", C.c_int32),
        ("cluster_id", C.c_int32),
    ]


class PpeTask(C.Structure):
    _fields_ = [
        ("mode", C.c_int32),
        ("clamp_low", C.c_int32),
        ("clamp_high", C.c_int32),
        ("lrelu_mult", C.c_int32),
        ("lrelu_shift", C.c_int32),
        ("has_quant", C.c_int32),
        ("quant_mult", C.c_int32),
        ("quant_shift", C.c_int32),
        ("quant_post_shift", C.c_int32),
        ("has_in_mult", C.c_int32),
        ("in1_quant_mult", C.c_int32),
        ("in2_quant_mult", C.c_int32),
        ("round_mode", C.c_int32),
        ("clamp_domain", C.c_int32),
    ]


class ClusterTaskDesc(C.Structure):
    _fields_ = [
        ("task_type", C.c_int32),
        ("flags", C.c_uint32),
        ("input", Tensor),
        ("weights", Tensor),
        ("weight_table", Tensor),
        ("output", Tensor),
        ("kernel_size", C.c_int32 * 2),
        ("kernel_strides", C.c_int32 * 2),
        ("kernel_pad_left", C.c_int32),
        ("kernel_pad_right", C.c_int32),
        ("kernel_pad_top", C.c_int32),
        ("kernel_pad_bottom", C.c_int32),
        ("variants", C.POINTER(DpuTask)),
        ("num_variants", C.c_uint32),
        ("reserved", C.c_uint32),
        ("ppe", C.POINTER(PpeTask)),
    ]


class ExecutorDesc(C.Structure):
    _fields_ = [("device_id", C.c_int32), ("log_level", C.c_int32)]


class Quant(C.Structure):
    _fields_ = [("scale", C.c_double), ("zero_point", C.c_int32), ("dtype", C.c_int32)]


# Every symbol the two headers declare: name -> (restype, argtypes)
_P = C.POINTER
class HwtestLayer(C.Structure):
    _fields_ = [
        ("present", C.c_int32),
        ("dtype", C.c_int32),
        ("dtype_name", C.c_char * 16),
        ("shape", C.c_int64 * 4),
        ("has_quant", C.c_int32),
        ("num_scales", C.c_int32),
        ("scale0", C.c_double),
        ("zero_point", C.c_int64),
        ("low_range", C.c_int64),
        ("high_range", C.c_int64),
        ("file_path", C.c_char * 256),
    ]


HWTEST_MAX_OUTPUTS = 8


class HwtestProgram(C.Structure):
    _fields_ = [
        ("num_tasks", C.c_int32),
        ("num_outputs", C.c_int32),
        ("num_intermediates", C.c_int32),
        ("outputs_identical", C.c_int32),
        ("output_shape", (C.c_int64 * 4) * HWTEST_MAX_OUTPUTS),
        ("intermediate_shape", C.c_int64 * 4),
    ]


class HwtestBinding(C.Structure):
    _fields_ = [
        ("input_tensor", C.c_int32),
        ("output_tensor", C.c_int32),
        ("weight_layer", C.c_int32),
        ("reserved", C.c_int32),
        ("input_offset_bytes", C.c_int64),
        ("output_offset_bytes", C.c_int64),
        ("weights_offset_bytes", C.c_int64),
    ]


class HwtestCase(C.Structure):
    _fields_ = [
        ("arch", C.c_int32),
        ("case_type", C.c_char * 48),
        ("task_type", C.c_int32),
        ("input", HwtestLayer),
        ("weight", HwtestLayer),
        ("output", HwtestLayer),
        ("kernel", C.c_int32 * 2),
        ("stride", C.c_int32 * 2),
        ("pad", C.c_int32 * 4),
        ("group", C.c_int32),
        ("dilation", C.c_int32),
        ("compress", C.c_int32),
        ("act_sparsity", C.c_int32),
        ("mpe_mode", C.c_int32),
        ("activation", C.c_int32),
        ("alpha", C.c_double),
        ("maximum", C.c_double),
        ("output_order", C.c_char * 8),
        ("ew_mode", C.c_char * 8),
    ]


class VpuipBuffer(C.Structure):
    _fields_ = [
        ("name", C.c_char * 32),
        ("section", C.c_int32),
        ("index", C.c_int32),
        ("byte_offset", C.c_int64),
        ("byte_size", C.c_int64),
        ("dtype", C.c_int32),
        ("elem_bytes", C.c_int32),
        ("zero_point", C.c_int32),
        ("dims", C.c_int64 * 4),
        ("strides_bytes", C.c_int64 * 4),
    ]


class VpuipInfo(C.Structure):
    _fields_ = [("num_buffers", C.c_int32), ("num_ops", C.c_int32), ("num_tasks", C.c_int32), ("num_dmas", C.c_int32),
                ("function", C.c_char * 64)]


# nce_vpuip_section_t / nce_vpuip_op_kind_t
VPUIP_ARGUMENT, VPUIP_CMX_NN, VPUIP_DDR, VPUIP_NETWORK_INPUT, VPUIP_NETWORK_OUTPUT = range(5)
VPUIP_OP_NCE_TASK, VPUIP_OP_DMA = 0, 1

# nce_hwtest_activation_t
HWTEST_ACT_NONE, HWTEST_ACT_RELU, HWTEST_ACT_RELUX, HWTEST_ACT_LEAKY_RELU, HWTEST_ACT_OTHER = range(5)

SYMBOLS = {
    "nceGetVersion": (C.c_int, [_P(C.c_uint32), _P(C.c_uint32)]),
    "nceExecutorCreate": (C.c_int, [ExecutorDesc, _P(C.c_void_p), _P(C.c_void_p)]),
    "nceExecutorDestroy": (C.c_int, [C.c_void_p]),
    "nceClusterTaskValidate": (C.c_int, [C.c_void_p, _P(ClusterTaskDesc)]),
    "nceClusterTaskEnqueue": (C.c_int, [C.c_void_p, _P(ClusterTaskDesc), C.c_void_p]),
    "nceTaskListCreate": (C.c_int, [C.c_void_p, _P(C.c_void_p)]),
    "nceTaskListAppend": (C.c_int, [C.c_void_p, _P(ClusterTaskDesc)]),
    "nceTaskListEnqueue": (C.c_int, [C.c_void_p, C.c_void_p]),
    "nceTaskListEnqueueNoAlloc": (C.c_int, [C.c_void_p, C.c_void_p]),
    "nceTaskListDestroy": (C.c_int, [C.c_void_p]),
    "nceExecutorSynchronize": (C.c_int, [C.c_void_p, C.c_void_p]),
    "nceLogHandleGetString": (C.c_int, [C.c_void_p, _P(C.c_size_t), C.c_char_p]),
    "nceQuantApproximate": (C.c_int, [C.c_int32, C.c_double, _P(C.c_int32), _P(C.c_int32), _P(C.c_int32)]),
    "nceEltwiseQuantApproximate": (C.c_int, [C.c_int32, C.c_double, C.c_double, C.c_double] + [_P(C.c_int32)] * 4),
    "ncePReLUApproximate": (C.c_int, [C.c_int32, C.c_double, _P(C.c_int32), _P(C.c_int32)]),
    "nceWeightsTableFill": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_double, C.c_double,
                                      _P(C.c_double), C.c_int32, _P(C.c_double), _P(C.c_int32)]),
    "ncePpeFromPostOp": (C.c_int, [C.c_int32, C.c_int32, C.c_double, C.c_double, Quant, _P(PpeTask)]),
    "ncePpeForAvgPool": (C.c_int, [C.c_int32, Quant, Quant, C.c_int32, C.c_int32, C.c_int32, C.c_double, C.c_double,
                                   _P(PpeTask)]),
    "ncePpeForEltwiseAdd": (C.c_int, [C.c_int32, Quant, Quant, Quant, C.c_int32, C.c_double, C.c_double, _P(PpeTask)]),
    "ncePpeFuseClamp": (C.c_int, [Quant, C.c_double, C.c_double, _P(PpeTask)]),
    "nceConvWeightSetBytes": (C.c_int, [C.c_int64, C.c_int64, C.c_int64, _P(C.c_int64), _P(C.c_int64)]),
    "nceWeightsTableCheck": (C.c_int, [_P(C.c_int32), C.c_int32, C.c_int32]),
    "nceHwtestParse": (C.c_int, [C.c_char_p, _P(C.c_void_p), C.c_void_p]),
    "nceHwtestDestroy": (C.c_int, [C.c_void_p]),
    "nceHwtestGetCase": (C.c_int, [C.c_void_p, _P(HwtestCase)]),
    "nceHwtestGetScales": (C.c_int, [C.c_void_p, C.c_int32, _P(C.c_double), C.c_int32]),
    "nceVpuipParse": (C.c_int, [C.c_char_p, _P(C.c_void_p), C.c_void_p]),
    "nceVpuipDestroy": (C.c_int, [C.c_void_p]),
    "nceVpuipGetInfo": (C.c_int, [C.c_void_p, _P(VpuipInfo)]),
    "nceVpuipGetBuffer": (C.c_int, [C.c_void_p, C.c_int32, _P(VpuipBuffer)]),
    "nceVpuipGetOp": (C.c_int, [C.c_void_p, C.c_int32, _P(C.c_int32), _P(C.c_int32)]),
    "nceVpuipBind": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_int64]),
    "nceVpuipGetTask": (C.c_int, [C.c_void_p, C.c_int32, _P(ClusterTaskDesc), C.c_void_p]),
    "nceVpuipEnqueue": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "nceHwtestBuildTask": (C.c_int, [C.c_void_p, _P(ClusterTaskDesc), _P(DpuTask), _P(PpeTask), _P(C.c_int32), C.c_int32,
                                     _P(C.c_int32), C.c_void_p]),
    "nceHwtestGetProgram": (C.c_int, [C.c_void_p, _P(HwtestProgram), C.c_void_p]),
    "nceHwtestBuildTaskAt": (C.c_int, [C.c_void_p, C.c_int32, _P(ClusterTaskDesc), _P(DpuTask), _P(PpeTask), _P(C.c_int32),
                                       C.c_int32, _P(C.c_int32), _P(HwtestBinding), C.c_void_p]),
}

_lib = None


def load_library():
    """Load libnce_hip.so (built in-tree by `make -C npu_plugin_amd/csrc` or __graft_entry__.build())."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP library first (python -c 'import __graft_entry__ as g; g.build()'). "
            "There is no CPU fallback.")
    # PyTorch ships its own HIP runtime (same SONAME as the system one). Two HIP runtimes in one process
    # do not share the GPU, so let torch load its copy first: the dynamic loader then binds this library
    # to the runtime that also owns the caller's tensors and streams.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
