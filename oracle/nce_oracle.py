"""ctypes binding of the CPU oracle (oracle/libnce_oracle.so). TEST INFRASTRUCTURE ONLY:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the package."""
import ctypes as C
import os
import subprocess

from npu_plugin_amd import _abi as abi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnce_oracle.so")
_lib = None
_P = C.POINTER


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "libnce_oracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        i32p = _P(C.c_int32)
        L.nce_oracle_approximate.argtypes = [C.c_int, C.c_double, _P(C.c_int64), i32p, i32p]
        L.nce_oracle_approximate.restype = None
        L.nce_oracle_quant_approx.argtypes = [C.c_int, C.c_double, i32p, i32p, i32p]
        L.nce_oracle_eltwise_approx.argtypes = [C.c_int, C.c_double, C.c_double, C.c_double, i32p, i32p, i32p, i32p]
        L.nce_oracle_prelu_approx.argtypes = [C.c_int, C.c_double, i32p, i32p]
        L.nce_oracle_scale_word.argtypes = [C.c_int, C.c_int32, C.c_int32, C.c_int32]
        L.nce_oracle_scale_word.restype = C.c_int32
        L.nce_oracle_float_bits.argtypes = [C.c_double]
        L.nce_oracle_float_bits.restype = C.c_int32
        L.nce_oracle_rescaled_bias.argtypes = [C.c_double, C.c_double, C.c_double, i32p]
        L.nce_oracle_weights_table.argtypes = [C.c_int, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_double,
                                               C.c_double, _P(C.c_double), C.c_int32, _P(C.c_double), C.c_int32, i32p]
        L.nce_oracle_avgpool_scale.argtypes = [C.c_double, C.c_double, C.c_int32, C.c_int32]
        L.nce_oracle_avgpool_scale.restype = C.c_double
        L.nce_oracle_ppe_stage1.argtypes = [C.c_int, C.c_int, C.c_double, C.c_double, C.c_int32, C.c_int32, C.c_double,
                                            C.c_int32, _P(abi.PpeTask)]
        L.nce_oracle_ppe_stage2_37xx.argtypes = [C.c_int, C.c_int32, C.c_int32, C.c_int32, _P(abi.PpeTask)]
        L.nce_oracle_ppe_stage2_37xx.restype = None
        L.nce_oracle_fuse_clamp_quant.argtypes = [C.c_double, C.c_int32, C.c_double, C.c_double, _P(C.c_int32), _P(C.c_int32)]
        L.nce_oracle_rshift_round.argtypes = [C.c_int64, C.c_int32, C.c_int32]
        L.nce_oracle_rshift_round.restype = C.c_int64
        L.nce_oracle_ppe.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P(abi.PpeTask), C.c_int32, C.c_int32]
        L.nce_oracle_ppe.restype = C.c_int32
        L.nce_oracle_run.argtypes = [_P(abi.ClusterTaskDesc), C.c_int]
        L.nce_oracle_max_threads.restype = C.c_int
        _lib = L
    return _lib


ARCH_30XX, ARCH_37XX = 0, 1


def approximate(bits, target):
    m, s, p = C.c_int64(), C.c_int32(), C.c_int32()
    lib().nce_oracle_approximate(bits, target, C.byref(m), C.byref(s), C.byref(p))
    return m.value, s.value, p.value


def quant_approx(target, arch=ARCH_37XX):
    m, s, p = C.c_int32(), C.c_int32(), C.c_int32()
    rc = lib().nce_oracle_quant_approx(arch, target, C.byref(m), C.byref(s), C.byref(p))
    if rc:
        raise ValueError("approximation refused")
    return m.value, s.value, p.value


def eltwise_approx(s1, s2, so, arch=ARCH_37XX):
    v = [C.c_int32() for _ in range(4)]
    rc = lib().nce_oracle_eltwise_approx(arch, s1, s2, so, *[C.byref(x) for x in v])
    if rc:
        raise ValueError("out of register range")
    return tuple(x.value for x in v)


def prelu_approx(alpha, arch=ARCH_37XX):
    m, s = C.c_int32(), C.c_int32()
    rc = lib().nce_oracle_prelu_approx(arch, alpha, C.byref(m), C.byref(s))
    if rc:
        raise ValueError("approximation refused")
    return m.value, s.value


def weights_table(oc, ptr_base, ptr_step, in_scale, out_scale, w_scales, bias=None, arch=ARCH_37XX,
                  sparsity_ptr=0xFFFFFF, lrelu_mult=-1):
    import numpy as np
    ws = (C.c_double * len(w_scales))(*w_scales)
    b = (C.c_double * oc)(*bias) if bias is not None else None
    out = np.zeros((oc, 4), dtype=np.int32)
    rc = lib().nce_oracle_weights_table(arch, oc, ptr_base, ptr_step, sparsity_ptr, in_scale, out_scale, ws,
                                        len(w_scales), b, lrelu_mult, out.ctypes.data_as(_P(C.c_int32)))
    if rc:
        raise ValueError("weights table refused")
    return out


def rshift_round(p, s, mode=0):
    return lib().nce_oracle_rshift_round(p, s, mode)


def ppe(acc, bias, mult, shift, ppe_struct, out_zp, out_dtype):
    return lib().nce_oracle_ppe(acc, bias, mult, shift, C.byref(ppe_struct) if ppe_struct is not None else None,
                                out_zp, out_dtype)


def run(task, nthreads=0):
    """task: npu_plugin_amd.NCEClusterTask whose buffers are HOST arrays (numpy)."""
    rc = lib().nce_oracle_run(C.byref(task.finalize()), nthreads)
    if rc:
        raise RuntimeError(f"oracle cannot evaluate this descriptor (code {rc})")
