"""Compiler-emitted VPUIP programs (textual MLIR) on the GPU executor.

    prog = vpuip.parse(open("program.mlir").read())
    prog.bind(vpuip.CMX_NN, 0, cmx)            # one buffer per (section, index): CMX per cluster, DDR, arguments
    prog.bind(vpuip.ARGUMENT, 0, network_input)
    prog.enqueue(executor, stream)             # NCE tasks and DMAs in program order

The parser and the conversion of VPUIP.NCEClusterTask to task descriptors live in the C library
(include/nce_vpuip.h); this module binds buffers and exposes the parsed tables.
"""
import ctypes as C

from . import _abi as abi
from .nce_task import Executor, NCEError, _address

ARGUMENT, CMX_NN, DDR, NETWORK_INPUT, NETWORK_OUTPUT = (abi.VPUIP_ARGUMENT, abi.VPUIP_CMX_NN, abi.VPUIP_DDR,
                                                       abi.VPUIP_NETWORK_INPUT, abi.VPUIP_NETWORK_OUTPUT)


class _Desc:
    """A descriptor resolved by the library, shaped like an NCEClusterTask for Executor / the oracle."""

    def __init__(self, desc, keep):
        self.desc = desc
        self._keep = keep

    def finalize(self):
        return self.desc


class Program:
    def __init__(self, handle, log_owner):
        self._lib = abi.load_library()
        self._h = handle
        self._log_owner = log_owner
        self._keep = {}
        info = abi.VpuipInfo()
        self._check(self._lib.nceVpuipGetInfo(self._h, C.byref(info)))
        self.function = info.function.decode()
        self.num_tasks, self.num_dmas = info.num_tasks, info.num_dmas
        self.buffers = []
        for i in range(info.num_buffers):
            b = abi.VpuipBuffer()
            self._check(self._lib.nceVpuipGetBuffer(self._h, i, C.byref(b)))
            self.buffers.append(b)
        self.ops = []
        for i in range(info.num_ops):
            kind, task = C.c_int32(), C.c_int32()
            self._check(self._lib.nceVpuipGetOp(self._h, i, C.byref(kind), C.byref(task)))
            self.ops.append((kind.value, task.value))

    def _check(self, rc):
        if rc != abi.SUCCESS:
            raise NCEError(rc, self._log_owner.log() if self._log_owner is not None else "")

    def buffer(self, name):
        for b in self.buffers:
            if b.name.decode() == name:
                return b
        raise KeyError(name)

    def section_size(self, section, index):
        """Bytes a binding of (section, index) must provide."""
        return max([b.byte_offset + b.byte_size for b in self.buffers if (b.section, b.index) == (section, index)] or [0])

    def bind(self, section, index, buf):
        nbytes = buf.numel() * buf.element_size() if hasattr(buf, "data_ptr") else buf.nbytes
        self._check(self._lib.nceVpuipBind(self._h, section, index, C.c_void_p(_address(buf)), nbytes))
        self._keep[(section, index)] = buf

    def task(self, i):
        """Descriptor of NCE task i with addresses resolved (usable with Executor.enqueue and the oracle)."""
        desc = abi.ClusterTaskDesc()
        self._check(self._lib.nceVpuipGetTask(self._h, i, C.byref(desc), self._log_owner._log))
        return _Desc(desc, self)

    def enqueue(self, executor, stream=None):
        rc = self._lib.nceVpuipEnqueue(self._h, executor._h, C.c_void_p(stream or 0))
        if rc != abi.SUCCESS:
            raise NCEError(rc, executor.log())

    def destroy(self):
        if self._h:
            self._lib.nceVpuipDestroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def parse(text):
    lib = abi.load_library()
    owner = Executor(device_id=-1, log_level=1)  # device-less: only owns the log for error text
    handle = C.c_void_p()
    rc = lib.nceVpuipParse(text.encode(), C.byref(handle), owner._log)
    if rc != abi.SUCCESS:
        raise NCEError(rc, owner.log())
    return Program(handle, owner)
