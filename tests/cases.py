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




def run_graph_oracle(graph, x, nthreads=0):
    """Every activation tensor of a ResNet50Graph computed by the oracle (host numpy buffers)."""
    from oracle import nce_oracle
    buffers = [np.zeros(s, dtype=np.uint8) for s in graph.tensors]
    buffers[0][...] = x
    weights = [L.weights for L in graph.layers]
    tables = [L.table for L in graph.layers]
    for task in graph.build_tasks(buffers, weights, tables):
        nce_oracle.run(task, nthreads)
    return buffers
