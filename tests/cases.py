"""Test-side view of the synthetic workloads: the package's generators plus the oracle runner."""
import numpy as np

from npu_plugin_amd.workloads import *  # noqa: F401,F403
from npu_plugin_amd.workloads import _np_dtype, build_task


def run_oracle(case, nthreads=0):
    from oracle import nce_oracle
    out = np.zeros(case.out_shape, dtype=_np_dtype(case.out_signed))
    task = build_task(case, case.input, case.weights, case.table, out)
    nce_oracle.run(task, nthreads)
    return out


