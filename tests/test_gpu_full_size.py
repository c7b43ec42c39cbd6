"""The benchmark configurations at their stated sizes, on the default dispatch (the instantiations bench.py times),
bit-exact against the CPU oracle. The dispatcher picks tile shapes, tiles per workgroup, index widths and the XCD
remap by size, so a batch-1 run does not cover them."""
import numpy as np
import pytest

from tests import cases as K
from tests.test_gpu_parity import check

pytestmark = pytest.mark.gpu


def test_cfg2_full_size(executor):
    check(K.cfg2(n=8), executor)


def test_cfg3_chain_full_size(executor):
    """depthwise 16x112x112x96 -> max pool -> average pool, each fed with the previous task's GPU output."""
    import torch
    dw = K.cfg3_dw(n=16)
    y_dw = K.run_oracle(dw)
    mp = K.cfg3_maxpool(n=16, x=y_dw)
    y_mp = K.run_oracle(mp)
    ap = K.cfg3_avgpool(n=16, x=y_mp)
    y_ap = K.run_oracle(ap)
    d_dw = K.DeviceCase(dw)
    d_mp = K.DeviceCase(mp)
    d_ap = K.DeviceCase(ap)
    t_mp = K.build_task(mp, d_dw.output, None, None, d_mp.output)
    t_ap = K.build_task(ap, d_mp.output, None, None, d_ap.output)
    tl = executor.task_list()
    for t in (d_dw.task, t_mp, t_ap):
        tl.append(t)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(2):  # the second pass replays the prepared launches
        for d in (d_dw, d_mp, d_ap):
            d.output.fill_(0x5A)
        tl.enqueue(stream)
        executor.synchronize(stream)
        assert np.array_equal(d_dw.output.cpu().numpy(), y_dw), "depthwise"
        assert np.array_equal(d_mp.output.cpu().numpy(), y_mp), "max pool"
        assert np.array_equal(d_ap.output.cpu().numpy(), y_ap), "average pool"
    tl.destroy()


def test_cfg4_full_size(executor):
    check(K.cfg4(n=16), executor)


def test_cfg5_batch32_every_tensor(executor):
    """The ResNet-50 graph at batch 32, 224 x 224: all 70 tensors against the oracle, on the first run of the task
    list (which prepares the launches) and on a replay."""
    import torch
    graph = K.ResNet50Graph(batch=32)
    x = graph.make_input()
    print("[case] resnet50 graph batch=32 size=224", flush=True)
    want = K.run_graph_oracle(graph, x)
    dg = K.DeviceGraph(graph, executor, x)
    stream = torch.cuda.current_stream().cuda_stream
    for rep in range(2):
        for buf in dg.buffers[1:]:
            buf.fill_(0x5A)
        dg.run(stream)
        executor.synchronize(stream)
        for L in graph.layers:
            got = dg.buffers[L.dst].cpu().numpy()
            assert np.array_equal(got, want[L.dst]), f"run {rep} {L.name}: {(got != want[L.dst]).sum()} bytes differ"
    assert len(np.unique(want[graph.output])) > 100, "degenerate network output"
    dg.task_list.destroy()


# The large-batch variants bench.py reports beside the configurations (the same layers with several rounds of work
# per CU): other tile shapes, tiles per workgroup and index widths than the configurations above.
def test_scaled_cfg2_batch512(executor):
    check(K.cfg2(n=512), executor)


def test_scaled_conv3x3_256_256(executor):
    check(K.conv_case(K.SEED + 20, 32, 56, 56, 256, 256, name="conv3x3_32x56x56x256_256"), executor)


def test_scaled_cfg3_dw_batch128(executor):
    check(K.cfg3_dw(n=128), executor)


def test_scaled_cfg3_maxpool_batch512(executor):
    check(K.cfg3_maxpool(n=512), executor)


def test_scaled_cfg4_batch512(executor):
    check(K.cfg4(n=512), executor)


def test_automatic_choice_of_the_tiled_kernel(executor, tuned):
    """Sizes at which the dispatcher itself picks the LDS-tiled kernel (long reduction, 256 or more output channels, two
    to four 128 x 128 workgroups per CU): same bytes as the oracle, and the same bytes as the weights-resident kernels
    (NCE_HIP_CONV_TILED=0) give."""
    import torch
    for case in (K.conv_case(K.SEED + 31, 8, 56, 56, 128, 256, name="conv3x3_8x56x56x128_256"),
                 K.conv_case(K.SEED + 32, 16, 28, 28, 1024, 512, k=(1, 1), pads=(0, 0, 0, 0), name="conv1x1_16x28x28x1024_512",
                             ppe=dict(mode=3, clamp_low=128, clamp_high=255))):
        want = K.run_oracle(case)
        got = K.run_hip(case, executor)
        assert np.array_equal(got, want), case.name
        assert np.array_equal(K.run_hip(case, tuned(NCE_HIP_CONV_TILED=0)), want), case.name + " (tiled kernel off)"
