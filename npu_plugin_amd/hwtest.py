"""The reference's single-operation test descriptors ("config.json" of its hwtest flow) on the GPU executor.

    case = hwtest.parse(open("config.json").read())      # nb::TestCaseJsonDescriptor
    task = case.build_task(input, weights, output)        # what buildSimpleZMajorConv & co. construct
    executor.enqueue(task)

Parsing and parameter generation happen in the C library (include/nce_hwtest.h); this module only binds
buffers to the descriptor it returns. Reference: src/vpux_translate_utils/src/hwtest/test_case_json_parser.cpp,
buildZMConvTest.cpp, buildDWConv.cpp, buildMaxPoolTest.cpp, buildAvgPoolTest.cpp, buildEltwiseTest.cpp.
"""
import ctypes as C

import numpy as np

from . import _abi as abi
from .nce_task import NCEClusterTask, NCEError, _address


def _log_text(lib, log):
    size = C.c_size_t(0)
    lib.nceLogHandleGetString(log, C.byref(size), None)
    buf = C.create_string_buffer(max(size.value, 1))
    lib.nceLogHandleGetString(log, C.byref(size), buf)
    return buf.value.decode(errors="replace")


class HwtestCase:
    """A parsed descriptor. Attribute names follow nb::TestCaseJsonDescriptor's layers."""

    def __init__(self, handle, info, log_source=None):
        self._lib = abi.load_library()
        self._handle = handle
        self.info = info
        self._log_source = log_source
        self.case_type = info.case_type.decode()
        self.task_type = info.task_type
        self.arch = info.arch
        self.output_order = info.output_order.decode()

    def scales(self, which):
        layer = (self.info.input, self.info.weight, self.info.output)[which]
        buf = (C.c_double * max(layer.num_scales, 1))()
        rc = self._lib.nceHwtestGetScales(self._handle, which, buf, layer.num_scales)
        if rc != abi.SUCCESS:
            raise NCEError(rc)
        return list(buf)[:layer.num_scales]

    def build_task(self, input, weights=None, output=None, executor=None):
        """Returns an NCEClusterTask whose attributes, variant, PPE task and weights table are the ones the
        reference's builder for this case type produces; `input`, `weights` (conv / depthwise weights in memory
        order, or the second eltwise operand) and `output` are caller-owned buffers (torch or numpy).
        The weights table is returned in `task.table` (numpy int32, host); pass `executor` to have it copied
        to the device the other buffers live on."""
        desc = abi.ClusterTaskDesc()
        variant = abi.DpuTask()
        ppe = abi.PpeTask()
        oc = int(self.info.output.shape[1])
        table = np.zeros((max(oc, 1), 4), dtype=np.int32)
        rows = C.c_int32(0)
        log = executor._log if executor is not None else None
        rc = self._lib.nceHwtestBuildTask(self._handle, C.byref(desc), C.byref(variant), C.byref(ppe),
                                          table.ctypes.data_as(C.POINTER(C.c_int32)), oc, C.byref(rows), log)
        if rc != abi.SUCCESS:
            raise NCEError(rc, executor.log() if executor is not None else "")
        task = NCEClusterTask(desc.task_type, None)
        task.desc = desc
        task._variants = [variant]
        task._ppe = ppe
        task.table = table[:rows.value] if rows.value else None
        task._keep = [input, weights, output]
        desc.input.data = _address(input)
        desc.output.data = _address(output)
        if weights is not None:
            desc.weights.data = _address(weights)
        if rows.value:
            dev_table = task.table
            if hasattr(input, "data_ptr"):  # torch: put the table where the activations are
                import torch
                dev_table = torch.from_numpy(task.table).to(input.device)
            task._keep.append(dev_table)
            desc.weight_table.data = _address(dev_table)
        task.finalize()
        return task

    def program(self, executor=None):
        """(num_tasks, output shapes, intermediate shape or None, outputs_identical) of the case's program: the case types
        the reference builds as several NCE tasks (DoubleZMajorConvolution, RaceConditionDPU, DifferentClustersDPU,
        MultiClustersDPU); a single-task case is a program of one task and one output."""
        g = abi.HwtestProgram()
        log = executor._log if executor is not None else None
        rc = self._lib.nceHwtestGetProgram(self._handle, C.byref(g), log)
        if rc != abi.SUCCESS:
            raise NCEError(rc, executor.log() if executor is not None else "")
        outs = [tuple(int(v) for v in g.output_shape[k]) for k in range(g.num_outputs)]
        mid = tuple(int(v) for v in g.intermediate_shape) if g.num_intermediates else None
        return g.num_tasks, outs, mid, bool(g.outputs_identical)

    def build_program(self, input, weights, outputs, intermediate=None, executor=None):
        """The case's tasks in program order. `weights`: one buffer per entry of the case's "weight" list; `outputs`: one
        buffer per output of program() (memory order: the case's output_order); `intermediate`: the tensor between the two
        convolutions of a DoubleZMajorConvolution (NHWC). Buffers are torch tensors or numpy arrays."""
        num_tasks, _, _, _ = self.program(executor)
        if not isinstance(weights, (list, tuple)):
            weights = [weights]
        tasks = []
        log = executor._log if executor is not None else None
        oc_max = max([int(self.info.output.shape[1]), int(self.info.weight.shape[0])] + [int(w.shape[0]) for w in weights if w is not None])
        for index in range(num_tasks):
            desc = abi.ClusterTaskDesc()
            variant = abi.DpuTask()
            ppe = abi.PpeTask()
            bind = abi.HwtestBinding()
            table = np.zeros((max(oc_max, 1), 4), dtype=np.int32)
            rows = C.c_int32(0)
            rc = self._lib.nceHwtestBuildTaskAt(self._handle, index, C.byref(desc), C.byref(variant), C.byref(ppe),
                                                table.ctypes.data_as(C.POINTER(C.c_int32)), oc_max, C.byref(rows), C.byref(bind), log)
            if rc != abi.SUCCESS:
                raise NCEError(rc, executor.log() if executor is not None else "")
            src = input if bind.input_tensor < 0 else intermediate
            dst = outputs[bind.output_tensor] if bind.output_tensor >= 0 else intermediate
            wts = weights[bind.weight_layer]
            if src is None or dst is None:
                raise ValueError("this case needs an intermediate tensor (see program())")
            task = NCEClusterTask(desc.task_type, None)
            task.desc = desc
            task._variants = [variant]
            task._ppe = ppe
            task.table = table[:rows.value] if rows.value else None
            task.binding = bind
            task._keep = [src, wts, dst]
            desc.input.data = _address(src) + bind.input_offset_bytes
            desc.output.data = _address(dst) + bind.output_offset_bytes
            desc.weights.data = _address(wts) + bind.weights_offset_bytes
            if rows.value:
                dev_table = task.table
                if hasattr(src, "data_ptr"):
                    import torch
                    dev_table = torch.from_numpy(task.table).to(src.device)
                task._keep.append(dev_table)
                desc.weight_table.data = _address(dev_table)
            task.finalize()
            tasks.append(task)
        return tasks

    def destroy(self):
        if self._handle:
            self._lib.nceHwtestDestroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def parse(json_text, executor=None):
    """Parse a descriptor; raises NCEError carrying the reference's message on malformed input."""
    lib = abi.load_library()
    handle = C.c_void_p()
    own_log = None
    log = executor._log if executor is not None else None
    if log is None:
        # a device-less executor only to own a log handle for the error text
        from .nce_task import Executor
        own_log = Executor(device_id=-1, log_level=1)
        log = own_log._log
    rc = lib.nceHwtestParse(json_text.encode(), C.byref(handle), log)
    if rc != abi.SUCCESS:
        raise NCEError(rc, _log_text(lib, log))
    info = abi.HwtestCase()
    rc = lib.nceHwtestGetCase(handle, C.byref(info))
    if rc != abi.SUCCESS:
        raise NCEError(rc)
    return HwtestCase(handle, info)
