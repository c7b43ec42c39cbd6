"""The C-ABI library loads and exports every symbol the headers declare (no GPU needed)."""
import ctypes
import os
import re

import npu_plugin_amd as nce
from npu_plugin_amd import _abi as abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    return set(re.findall(r"^nce_result_t\s+(nce\w+)\s*\(", text, flags=re.M))


def test_every_declared_symbol_is_exported_and_bound():
    declared = _declared("nce_hip.h") | _declared("nce_params.h") | _declared("nce_hwtest.h") | _declared("nce_vpuip.h")
    assert len(declared) >= 28
    lib = abi.load_library()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported by libnce_hip.so"
    assert declared == set(abi.SYMBOLS), "ctypes table and headers disagree"


def test_struct_sizes_match_the_header_layout():
    # 8-byte pointer + 2 x int32 + 8 x int64
    assert ctypes.sizeof(abi.Tensor) == 8 + 8 + 64
    assert ctypes.sizeof(abi.DpuTask) == 12 * 4
    assert ctypes.sizeof(abi.PpeTask) == 14 * 4
    assert ctypes.sizeof(abi.ClusterTaskDesc) == 8 + 4 * 80 + 8 * 4 + 8 + 8 + 8


def test_version_and_null_handles():
    lib = abi.load_library()
    major, minor = ctypes.c_uint32(), ctypes.c_uint32()
    assert lib.nceGetVersion(ctypes.byref(major), ctypes.byref(minor)) == abi.SUCCESS
    assert (major.value, minor.value) == (0, 1)
    assert lib.nceExecutorDestroy(None) == abi.ERROR_INVALID_NULL_HANDLE
    assert lib.nceClusterTaskValidate(None, None) == abi.ERROR_INVALID_NULL_HANDLE
    assert lib.nceClusterTaskEnqueue(None, None, None) == abi.ERROR_INVALID_NULL_HANDLE
    assert lib.nceLogHandleGetString(None, None, None) == abi.ERROR_INVALID_NULL_HANDLE


def test_deviceless_executor_validates_but_refuses_to_launch(validator):
    import numpy as np
    from tests.cases import build_task, cfg1
    case = cfg1()
    out = np.zeros(case.out_shape, dtype=np.uint8)
    task = build_task(case, case.input, case.weights, case.table, out)
    validator.validate(task)
    try:
        validator.enqueue(task)
    except nce.NCEError as e:
        assert e.code == abi.ERROR_UNSUPPORTED and "without a device" in e.log
    else:
        raise AssertionError("a device-less executor must not launch")
    assert not out.any(), "nothing may have been computed on the CPU"
