"""Persistent segments of a task list (NCE_HIP_PERSISTENT=1): runs of weights-resident convolutions as one launch of 256
workgroups with XCD-local barriers between the layers. Every tensor of the ResNet-50 graph must equal the oracle's."""
import os

import numpy as np
import pytest

from tests import cases as K

pytestmark = pytest.mark.gpu


def _executor(**env):
    """An executor created under the given environment (its knobs are read once, at creation)."""
    import npu_plugin_amd as nce
    saved = {k: os.environ.get(k) for k in env}
    os.environ.update(env)
    try:
        return nce.Executor(device_id=0, log_level=3)
    finally:
        for k, v in saved.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v


@pytest.mark.parametrize("batch,size", [(8, 64), (16, 96)])
def test_resnet50_graph_persistent(tuned, batch, size):
    import torch
    executor = _executor(NCE_HIP_PERSISTENT="1")
    graph = K.ResNet50Graph(batch=batch, size=size)
    x = graph.make_input()
    print(f"[case] resnet50 graph persistent batch={batch} size={size}", flush=True)
    want = K.run_graph_oracle(graph, x)
    dg = K.DeviceGraph(graph, executor, x)
    stream = torch.cuda.current_stream().cuda_stream
    for rep in range(3):
        print(f"[run] {rep}", flush=True)
        dg.run(stream)
        executor.synchronize(stream)
        for L in graph.layers:
            got = dg.buffers[L.dst].cpu().numpy()
            assert np.array_equal(got, want[L.dst]), f"run {rep} {L.name}: {(got != want[L.dst]).sum()} bytes differ"
    text = executor.log()
    print(text[-1500:], flush=True)
    assert "persistent launch" in text, "no persistent segment was formed"
    dg.task_list.destroy()


def test_persistent_wait_limit_reports_and_falls_back(tuned):
    """A wait limit of zero makes the segment's first unsatisfied wait give up (every workgroup still leaves the kernel
    normally): the synchronise call must report the failure, and the next enqueue - persistent launches now off for
    the executor - must produce the oracle's tensors through ordinary launches."""
    import torch
    import npu_plugin_amd as nce
    executor = _executor(NCE_HIP_PERSISTENT="1", NCE_HIP_PERSISTENT_WAIT_US="0")
    graph = K.ResNet50Graph(batch=8, size=64)
    x = graph.make_input()
    print("[case] resnet50 graph persistent, wait limit 0", flush=True)
    want = K.run_graph_oracle(graph, x)
    dg = K.DeviceGraph(graph, executor, x)
    stream = torch.cuda.current_stream().cuda_stream
    dg.run(stream)
    with pytest.raises(nce.NCEError, match="did not complete"):
        executor.synchronize(stream)
    print("[run] after the failure", flush=True)
    dg.run(stream)
    executor.synchronize(stream)
    for L in graph.layers:
        got = dg.buffers[L.dst].cpu().numpy()
        assert np.array_equal(got, want[L.dst]), f"{L.name}: {(got != want[L.dst]).sum()} bytes differ"
    dg.task_list.destroy()
