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


# (32, 224) is the size the benchmark times (four images per XCD: the kernel variants the full-size layers use)
@pytest.mark.parametrize("batch,size", [(8, 64), (16, 96), (32, 224)])
def test_resnet50_graph_persistent(batch, size):
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


def test_persistent_wait_limit_reports_and_falls_back():
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


def _arena_buffers(graph, device="cuda:0"):
    """The graph's activation tensors placed in ONE arena the way a memory planner would: a tensor's bytes are free again
    after its last reader, and later tensors - of other shapes, hence other batch strides - take them (first fit, 256-byte
    granules). Layers of a persistent segment run ahead of each other per XCD, so such reuse inside a segment would corrupt
    data: the segment builder has to see the overlap and cut the segment there."""
    import torch
    last_use = {}
    for j, L in enumerate(graph.layers):
        for t in (L.src, L.src2, L.dst):
            if t >= 0:
                last_use[t] = j
    last_use[graph.output] = len(graph.layers)
    born = {0: -1}
    for j, L in enumerate(graph.layers):
        born[L.dst] = j
    size = {t: (int(np.prod(s)) + 255) // 256 * 256 for t, s in enumerate(graph.tensors)}
    placed = {}      # tensor -> (offset, size)
    order = sorted(born, key=lambda t: born[t])
    total = 0
    for t in order:
        live = [(o, s) for u, (o, s) in placed.items() if last_use[u] >= born[t]]   # (a layer's inputs outlive its output's birth)
        live.sort()
        off = 0
        for o, s in live:
            if off + size[t] <= o:
                break
            off = max(off, o + s)
        placed[t] = (off, size[t])
        total = max(total, off + size[t])
    arena = torch.zeros(total, dtype=torch.uint8, device=device)
    bufs = []
    for t, shape in enumerate(graph.tensors):
        off, _ = placed[t]
        bufs.append(arena[off:off + int(np.prod(shape))].view(*shape))
    shared = sum(s for _, s in placed.values()) - total
    return arena, bufs, shared


@pytest.mark.parametrize("no_alloc", [False, True])
def test_persistent_with_reused_activation_memory(no_alloc):
    """Activations in a planner-style arena (tensors reuse each other's bytes): persistent segments must stop where two
    layers would touch the same bytes in different batch shares. The network output must equal the oracle's."""
    import torch
    executor = _executor(NCE_HIP_PERSISTENT="1")
    graph = K.ResNet50Graph(batch=16, size=64)
    x = graph.make_input()
    print(f"[case] resnet50 graph in an arena, persistent, no_alloc={no_alloc}", flush=True)
    want = K.run_graph_oracle(graph, x)
    arena, bufs, shared = _arena_buffers(graph)
    assert shared > 0, "the arena does not reuse any memory"
    bufs[0].copy_(torch.from_numpy(x))
    weights = [torch.from_numpy(L.weights).to("cuda:0") if L.weights is not None else None for L in graph.layers]
    tables = [torch.from_numpy(L.table).to("cuda:0") if L.table is not None else None for L in graph.layers]
    tasks = graph.build_tasks(bufs, weights, tables)
    tl = executor.task_list()
    for t in tasks:
        tl.append(t)
    stream = torch.cuda.current_stream().cuda_stream
    for rep in range(3):
        bufs[0].copy_(torch.from_numpy(x))  # (the input's bytes may have been reused too)
        torch.cuda.synchronize()
        (tl.enqueue_no_alloc if no_alloc else tl.enqueue)(stream)
        executor.synchronize(stream)
        got = bufs[graph.output].cpu().numpy()
        assert np.array_equal(got, want[graph.output]), f"run {rep}: {(got != want[graph.output]).sum()} bytes of the output differ"
    text = executor.log()
    print(text[-800:], flush=True)
    assert "persistent launch" in text, "no persistent segment was formed"
    tl.destroy()
