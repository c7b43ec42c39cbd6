"""Where the time of the ResNet-50 task graph goes, launch by launch: reads the timestamps that a probe build of the
library (`make -C npu_plugin_amd/csrc probe`) writes from inside the weights-resident convolution kernel - kernel entry,
requests issued, before / after the workgroup barrier, start of the reduction loop, end of the last tile's loop, exit; the
100 MHz wall clock every wave reads with s_memrealtime - during one step of the graph, and prints per convolution the gap
to the launch before it and the medians over its waves.

    python3 -m npu_plugin_amd.probe_timeline [batch]

Every convolution runs on the kernel that carries the marks (NCE_HIP_CONV_PATCH=0, NCE_HIP_CONV_TILED=0). A launch records
the workgroups 0..255 of its first grid dimension; slices of one pixel group overwrite each other, so figures below about
0.3 us are not resolved."""
import ctypes as C
import os
import sys

import numpy as np

from . import _abi as abi


def main(batch=32):
    here = os.path.dirname(os.path.abspath(__file__))
    abi.LIB_PATH = os.path.join(here, "libnce_hip_probe.so")
    os.environ["NCE_HIP_CONV_PATCH"] = "0"
    os.environ["NCE_HIP_CONV_TILED"] = "0"
    import torch
    from . import Executor
    from . import workloads as W
    ex = Executor(device_id=0)
    lib = abi.load_library()
    lib.nceProbeSetWresTrace.argtypes = [C.c_void_p]
    lib.nceProbeSetWresTrace.restype = None
    graph = W.ResNet50Graph(batch=batch)
    trace = torch.zeros(64 * 256 * 8 * 8, dtype=torch.int64, device="cuda")
    lib.nceProbeSetWresTrace(trace.data_ptr())   # before the task list is built: a list keeps its launch arguments
    dg = W.DeviceGraph(graph, ex, graph.make_input())
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(50):
        dg.run(stream)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        dg.run(stream)
    e1.record()
    torch.cuda.synchronize()
    print(f"step {e0.elapsed_time(e1) / 20 * 1000:.1f} us (probe build, marks on)")
    trace.zero_()
    torch.cuda.synchronize()
    dg.run(stream)
    torch.cuda.synchronize()
    t = trace.cpu().numpy().reshape(64, 256, 8, 8).astype(np.float64) / 100.0   # us
    convs = [L for L in graph.layers if L.task_type == 0]
    print("gap = first entry - previous launch's last exit; then, from the launch's first entry, medians over its waves (us):")
    print(f"{'launch':26s} {'gap':>5s} | {'entry':>5s} {'req':>5s} {'bar':>5s} {'after':>5s} {'loop':>5s} {'l.end':>6s} {'exit':>6s} {'last':>6s}")
    prev_end = None
    keys = ("gap", "req", "bar", "after", "loop", "lend", "exit", "last")
    tot = dict.fromkeys(keys, 0.0)
    for i, L in enumerate(convs):
        r = t[i]
        used = r[:, :, 0] > 0
        if not used.any():
            print(f"{L.name:26s} (no marks: another kernel took it)")
            prev_end = None
            continue
        t0 = r[:, :, 0][used].min()

        def med(k):
            v = r[:, :, k][used & (r[:, :, k] > 0)]
            return (np.median(v) - t0) if v.size else float("nan")
        end = r[:, :, 6][used & (r[:, :, 6] > 0)].max()
        gap = (t0 - prev_end) if prev_end is not None else 0.0
        prev_end = end
        row = dict(gap=gap, req=med(1), bar=med(2), after=med(3), loop=med(4), lend=med(5), exit=med(6), last=end - t0)
        for k in keys:
            tot[k] += row[k]
        print(f"{L.name:26s} {gap:5.2f} | {med(0):5.2f} {row['req']:5.2f} {row['bar']:5.2f} {row['after']:5.2f} {row['loop']:5.2f} "
              f"{row['lend']:6.2f} {row['exit']:6.2f} {row['last']:6.2f}")
    print("sums over the convolutions (us): " + ", ".join(f"{k} {v:.1f}" for k, v in tot.items()))
    dg.task_list.destroy()
    ex.destroy()


if __name__ == "__main__":
    main(int(sys.argv[1]) if len(sys.argv) > 1 else 32)
