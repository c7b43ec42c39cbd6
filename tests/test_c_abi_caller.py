"""A C99 program compiled against include/*.h and linked with libnce_hip.so (no GPU needed), and one executor driven
from several host threads at once."""
import os
import subprocess
import threading

import numpy as np

import npu_plugin_amd as nce
from npu_plugin_amd import _abi as abi
from tests import cases as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c99_caller_builds_links_and_validates_cfg1(tmp_path):
    exe = str(tmp_path / "cfg1_validate")
    libdir = os.path.dirname(abi.LIB_PATH)
    cmd = ["gcc", "-std=c99", "-pedantic-errors", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "c_caller", "cfg1_validate.c"), "-o", exe, "-L", libdir, "-l:" + os.path.basename(abi.LIB_PATH),
           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stdout + r.stderr


def test_one_executor_from_four_threads():
    """Validate and task-list Append on ONE executor from four threads at once (the reference's compiler handle is used
    the same way, src/vpux_driver_compiler/test/functional/vcl_tests_parallel_compilation.cpp): every call returns what
    it returns single-threaded and the log holds one line per rejected descriptor."""
    ex = nce.Executor(device_id=-1, log_level=1)
    good = K.cfg1()
    bad = K.conv_case(3, 1, 8, 8, 16, 16, k=(3, 3))
    bad.kernel = (3, 12)   # kernel width above the limit
    errors, rejected = [], [0] * 4

    def worker(i):
        try:
            out = np.zeros(good.out_shape, dtype=np.uint8)
            tg = K.build_task(good, good.input, good.weights, good.table, out)
            tb = K.build_task(bad, bad.input, np.zeros((16, 3, 12, 16), np.int8), bad.table, np.zeros(bad.out_shape, dtype=np.uint8))
            tl = ex.task_list()
            for _ in range(200):
                assert ex.validate_code(tg) == abi.SUCCESS
                if ex.validate_code(tb) != abi.SUCCESS:
                    rejected[i] += 1
                tl.append(tg)
            tl.destroy()
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert rejected == [200] * 4
    lines = [ln for ln in ex.log().splitlines() if ln]
    assert len(lines) == 800 and all("kernel width" in ln for ln in lines)
    ex.destroy()
