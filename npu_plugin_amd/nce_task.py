"""Host-side mirror of the reference's NCE task interface, over the C-ABI of include/nce_hip.h.

Names follow the reference so that a test reads like one of its hwtest builders
(src/vpux_translate_utils/src/hwtest/buildZMConvTest.cpp:352-401):

    task = NCEClusterTask(TASK_CONV, input, weights, weight_table, output,
                          kernel_size=[3, 3], kernel_strides=[1, 1], kernel_padding=(1, 1, 1, 1))
    task.addDPUTask(outStart, outEnd, pad)              # VPUIP::NCEClusterTaskOp::addDPUTask
    task.addPPETask(PPE_LPRELU, clamp_low, clamp_high, lrelu_mult, lrelu_shift)   # ...::addPPETask
    executor.enqueue(task)

Buffers are anything with a device (or host) address: torch tensors and numpy arrays both work,
the library itself only ever sees raw pointers.
"""
import ctypes as C

from . import _abi as abi
from ._abi import *  # noqa: F401,F403  (re-export the enums)


class NCEError(RuntimeError):
    def __init__(self, code, log=""):
        self.code = code
        self.log = log
        super().__init__(f"{abi.RESULT_NAMES.get(code, hex(code))}: {log.strip()}")


def _address(buf):
    if hasattr(buf, "data_ptr"):  # torch
        return buf.data_ptr()
    return buf.ctypes.data  # numpy


def _shape_strides_bytes(buf):
    if hasattr(buf, "data_ptr"):
        es = buf.element_size()
        return tuple(buf.shape), tuple(s * es for s in buf.stride())
    return tuple(buf.shape), tuple(buf.strides)


def _dtype_code(buf):
    name = str(buf.dtype).replace("torch.", "")
    try:
        return {"uint8": abi.DT_U8, "int8": abi.DT_I8, "int32": abi.DT_SI32}[name]
    except KeyError:
        raise TypeError(f"unsupported element type {buf.dtype}") from None


def _tensor(buf, dims, strides, zero_point):
    t = abi.Tensor()
    t.data = _address(buf)
    t.dtype = _dtype_code(buf)
    t.zero_point = int(zero_point)
    t.dims = (C.c_int64 * 4)(*[int(d) for d in dims])
    t.strides_bytes = (C.c_int64 * 4)(*[int(s) for s in strides])
    return t


def activation(buf, zero_point=0):
    """buf: array of shape (N, H, W, C) = NHWC memory order. Logical dims are [N, C, H, W]."""
    (n, h, w, c), (sn, sh, sw, sc) = _shape_strides_bytes(buf)
    return _tensor(buf, [n, c, h, w], [sn, sc, sh, sw], zero_point), buf


def conv_weights(buf, zero_point=0):
    """buf: array of shape (OC, KY, KX, IC) = OYXI memory order. Logical dims are [OC, IC, KY, KX]."""
    (oc, ky, kx, ic), (so, sy, sx, si) = _shape_strides_bytes(buf)
    return _tensor(buf, [oc, ic, ky, kx], [so, si, sy, sx], zero_point), buf


def depthwise_weights(buf, zero_point=0):
    """buf: array of shape (C, 16*k): one row per channel, KY*KX taps row-major then zero padding."""
    (c, row), (sc, sb) = _shape_strides_bytes(buf)
    return _tensor(buf, [c, row, 1, 1], [sc, sb, sb, sb], zero_point), buf


def weight_table(buf):
    """buf: int32 array of shape (OC, 4): {weights ptr, sparsity ptr, (mult<<16)|(shift<<8), bias}."""
    (oc, four), (so, se) = _shape_strides_bytes(buf)
    assert four == 4
    return _tensor(buf, [oc, 1, 1, 4], [so, 4 * se, 4 * se, se], 0), buf


class NCEClusterTask:
    """One VPUIP.NCEClusterTask: operands + attributes + DPUTask variants + PPETask
    (src/vpux_compiler/tblgen/vpux/compiler/dialect/VPUIP/ops.td:2783-2831)."""

    def __init__(self, task_type, input, weights=None, weight_table=None, output=None, kernel_size=None,
                 kernel_strides=None, kernel_padding=(0, 0, 0, 0), flags=0):
        self.task_type = task_type
        self._keep = []
        self.desc = abi.ClusterTaskDesc()
        self.desc.task_type = task_type
        self.desc.flags = flags
        for name, op in (("input", input), ("weights", weights), ("weight_table", weight_table), ("output", output)):
            if op is not None:
                t, buf = op
                setattr(self.desc, name, t)
                self._keep.append(buf)
        if kernel_size is not None:
            self.desc.kernel_size = (C.c_int32 * 2)(*kernel_size)
        if kernel_strides is not None:
            self.desc.kernel_strides = (C.c_int32 * 2)(*kernel_strides)
        left, right, top, bottom = kernel_padding  # VPU::PaddingAttr order
        self.desc.kernel_pad_left, self.desc.kernel_pad_right = left, right
        self.desc.kernel_pad_top, self.desc.kernel_pad_bottom = top, bottom
        self._variants = []
        self._ppe = None

    def addDPUTask(self, outStart, outEnd, pad=(0, 0, 0, 0), mpeMode=abi.MPE_CUBOID_16x16, clusterId=0):
        """outStart / outEnd: [x, y, z] inclusive; pad: (left, right, top, bottom)
        (src/vpux_compiler/src/dialect/VPUIP/ops/nce_cluster_task.cpp:272-297)."""
        d = abi.DpuTask()
        d.out_start = (C.c_int32 * 3)(*outStart)
        d.out_end = (C.c_int32 * 3)(*outEnd)
        d.pad_left, d.pad_right, d.pad_top, d.pad_bottom = pad
        d.mpe_mode = mpeMode
        d.cluster_id = clusterId
        self._variants.append(d)
        return d

    def addWholeOutputDPUTask(self, mpeMode=abi.MPE_CUBOID_16x16):
        """One variant covering the whole output carrying the full kernel padding, as the hwtest
        builders do (src/vpux_translate_utils/src/hwtest/buildZMConvTest.cpp:360-371)."""
        o = self.desc.output
        d = self.desc
        return self.addDPUTask([0, 0, 0], [o.dims[3] - 1, o.dims[2] - 1, o.dims[1] - 1],
                               (d.kernel_pad_left, d.kernel_pad_right, d.kernel_pad_top, d.kernel_pad_bottom), mpeMode)

    def addPPETask(self, mode=abi.PPE_NOOP, clamp_low=abi.INT32_MIN, clamp_high=abi.INT32_MAX, lrelu_mult=1,
                   lrelu_shift=0, quant_mult=None, quant_shift=None, quant_post_shift=0, in1_quant_mult=None,
                   in2_quant_mult=None, round_mode=abi.ROUND_HALF_UP, clamp_domain=abi.CLAMP_POST_ZP):
        """nce_cluster_task.cpp:299-341 (argument order of the reference's addPPETask)."""
        p = abi.PpeTask()
        p.mode = mode
        p.clamp_low, p.clamp_high = clamp_low, clamp_high
        p.lrelu_mult, p.lrelu_shift = lrelu_mult, lrelu_shift
        p.has_quant = int(quant_mult is not None)
        p.quant_mult = quant_mult if quant_mult is not None else 1
        p.quant_shift = quant_shift if quant_shift is not None else 0
        p.quant_post_shift = quant_post_shift
        p.has_in_mult = int(in1_quant_mult is not None)
        p.in1_quant_mult = in1_quant_mult if in1_quant_mult is not None else 1
        p.in2_quant_mult = in2_quant_mult if in2_quant_mult is not None else 1
        p.round_mode = round_mode
        p.clamp_domain = clamp_domain
        self._ppe = p
        return p

    def setPPE(self, ppe_struct):
        """Attach a PpeTask filled by the nce_params.h generators."""
        self._ppe = ppe_struct

    def finalize(self):
        """Materialise the variant array and PPE pointer; returns the ctypes descriptor."""
        n = len(self._variants)
        self._variant_array = (abi.DpuTask * max(n, 1))(*self._variants)
        self.desc.variants = C.cast(self._variant_array, C.POINTER(abi.DpuTask)) if n else None
        self.desc.num_variants = n
        self.desc.ppe = C.pointer(self._ppe) if self._ppe is not None else None
        return self.desc


class TaskList:
    def __init__(self, executor):
        self._ex = executor
        self._lib = executor._lib
        self._h = C.c_void_p()
        executor._check(self._lib.nceTaskListCreate(executor._h, C.byref(self._h)))
        self._keep = []

    def append(self, task):
        self._keep.append(task)
        self._ex._check(self._lib.nceTaskListAppend(self._h, C.byref(task.finalize())))

    def enqueue(self, stream=None):
        self._ex._check(self._lib.nceTaskListEnqueue(self._h, C.c_void_p(stream or 0)))

    def enqueue_no_alloc(self, stream=None):
        """nceTaskListEnqueueNoAlloc: the same launches with no device allocation (the library's fixed workspace)."""
        self._ex._check(self._lib.nceTaskListEnqueueNoAlloc(self._h, C.c_void_p(stream or 0)))

    def destroy(self):
        if self._h:
            self._lib.nceTaskListDestroy(self._h)
            self._h = C.c_void_p()


class Executor:
    """nceExecutorCreate / Enqueue / Synchronize. device_id < 0 gives a validate-only executor."""

    def __init__(self, device_id=0, log_level=2):
        self._lib = abi.load_library()
        self._h = C.c_void_p()
        self._log = C.c_void_p()
        rc = self._lib.nceExecutorCreate(abi.ExecutorDesc(device_id, log_level), C.byref(self._h), C.byref(self._log))
        if rc != abi.SUCCESS:
            raise NCEError(rc, f"nceExecutorCreate(device_id={device_id}) failed; a GPU is required, there is no CPU fallback")

    def log(self):
        size = C.c_size_t(0)
        self._lib.nceLogHandleGetString(self._log, C.byref(size), None)
        buf = C.create_string_buffer(size.value)
        self._lib.nceLogHandleGetString(self._log, C.byref(size), buf)
        return buf.value.decode()

    def _check(self, rc):
        if rc != abi.SUCCESS:
            raise NCEError(rc, self.log())

    def validate_code(self, task):
        return self._lib.nceClusterTaskValidate(self._h, C.byref(task.finalize()))

    def validate(self, task):
        self._check(self.validate_code(task))

    def enqueue(self, task, stream=None):
        self._check(self._lib.nceClusterTaskEnqueue(self._h, C.byref(task.finalize()), C.c_void_p(stream or 0)))

    def synchronize(self, stream=None):
        self._check(self._lib.nceExecutorSynchronize(self._h, C.c_void_p(stream or 0)))

    def task_list(self):
        return TaskList(self)

    def destroy(self):
        if self._h:
            self._lib.nceExecutorDestroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
