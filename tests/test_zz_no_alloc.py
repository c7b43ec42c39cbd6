"""nceTaskListEnqueueNoAlloc: the enqueue form that allocates nothing on the device (its persistent launches keep their
tables and counters in the library's fixed workspace). Its tensors must equal, byte for byte, those of nceTaskListEnqueue
on an executor with persistent launches on - on calls in a row with a larger and then a smaller graph, which share the
workspace - and the oracle's."""
import os

import numpy as np
import pytest

from tests import cases as K

pytestmark = pytest.mark.gpu


def _executor(**env):
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


def _tensors(dg, graph):
    return {L.dst: dg.buffers[L.dst].cpu().numpy() for L in graph.layers}


def test_no_alloc_enqueue_matches_enqueue():
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    ex_ref = _executor(NCE_HIP_PERSISTENT="1")
    ex = _executor()
    cases = []
    for batch, size in [(16, 96), (8, 64)]:  # the second call's graph is the smaller one
        graph = K.ResNet50Graph(batch=batch, size=size)
        x = graph.make_input()
        print(f"[case] reference run, batch={batch} size={size}", flush=True)
        dg_ref = K.DeviceGraph(graph, ex_ref, x)
        dg_ref.run(stream)
        ex_ref.synchronize(stream)
        want = _tensors(dg_ref, graph)
        oracle = K.run_graph_oracle(graph, x)
        for dst, t in want.items():
            assert np.array_equal(t, oracle[dst])
        dg_ref.task_list.destroy()
        cases.append((graph, K.DeviceGraph(graph, ex, x), want))
    assert "persistent launch" in ex_ref.log()

    order = [0, 1, 0, 1]
    for call, k in enumerate(order):
        graph, dg, want = cases[k]
        for L in graph.layers:
            dg.buffers[L.dst].zero_()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        print(f"[run] no-alloc call {call}: batch={graph.batch}", flush=True)
        dg.task_list.enqueue_no_alloc(stream)
        ex.synchronize(stream)
        free_after = torch.cuda.mem_get_info()[0]
        got = _tensors(dg, graph)
        for L in graph.layers:
            assert np.array_equal(got[L.dst], want[L.dst]), f"call {call} {L.name}: {(got[L.dst] != want[L.dst]).sum()} bytes differ"
        if call >= 2:  # (the first calls may load code objects)
            assert free_after == free_before, f"call {call}: device memory in use changed by {free_before - free_after} bytes"
    text = ex.log()
    assert "fixed workspace" in text, "no persistent launch used the fixed workspace"
    for _, dg, _ in cases:
        dg.task_list.destroy()


def test_no_alloc_enqueue_rejects_more_layers_than_the_workspace_holds():
    import torch
    import npu_plugin_amd as nce
    stream = torch.cuda.current_stream().cuda_stream
    ex = _executor()
    graph = K.ResNet50Graph(batch=8, size=64)
    dg = K.DeviceGraph(graph, ex, graph.make_input())
    for _ in range(3):  # the same tasks three more times: far more layers in persistent launches than the 64 the workspace holds
        for t in dg.tasks:
            dg.task_list.append(t)
    print("[case] no-alloc enqueue of an over-long list", flush=True)
    with pytest.raises(nce.NCEError, match="limit of the fixed workspace") as info:
        dg.task_list.enqueue_no_alloc(stream)
    assert info.value.code == 0x78000008  # NCE_RESULT_ERROR_UNSUPPORTED
    dg.task_list.enqueue(stream)  # the allocating form takes the list
    ex.synchronize(stream)
    dg.task_list.destroy()
