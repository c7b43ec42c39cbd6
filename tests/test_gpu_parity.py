"""Parity of the HIP executor with the CPU oracle, through the C-ABI, bit-exact (integer path)."""
import numpy as np
import pytest

import npu_plugin_amd as nce
from tests import cases as K

pytestmark = pytest.mark.gpu


def check(case, executor):
    print(f"[case] {case.name} in={case.input.shape} out={case.out_shape}", flush=True)
    want = K.run_oracle(case)
    got = K.run_hip(case, executor)
    bad = np.argwhere(want != got)
    assert bad.size == 0, (f"{case.name}: {len(bad)} of {want.size} bytes differ; first at {bad[0].tolist()} "
                           f"oracle={want[tuple(bad[0])]} hip={got[tuple(bad[0])]}")


# ---- the five task types at small sizes ------------------------------------------------------

def test_cfg1_conv(executor):
    check(K.cfg1(), executor)


def test_cfg2_conv_lrelu_small_batch(executor):
    check(K.cfg2(n=1), executor)


@pytest.mark.parametrize("ic,oc", [(16, 16), (32, 48), (64, 64), (48, 144), (128, 80), (16, 272)])
def test_conv_channel_shapes(executor, ic, oc):
    check(K.conv_case(10 + ic + oc, 2, 9, 11, ic, oc), executor)


@pytest.mark.parametrize("k,s,pads", [((1, 1), (1, 1), (0, 0, 0, 0)), ((1, 1), (2, 2), (0, 0, 0, 0)),
                                      ((3, 3), (2, 2), (1, 1, 1, 1)), ((3, 3), (2, 2), (0, 1, 0, 1)),
                                      ((7, 7), (2, 2), (3, 3, 3, 3)), ((5, 3), (1, 2), (1, 1, 2, 2)),
                                      ((11, 11), (4, 4), (5, 5, 5, 5)), ((2, 2), (1, 1), (1, 0, 1, 0)),
                                      ((1, 1), (1, 1), (1, 1, 1, 1)), ((3, 1), (8, 1), (0, 0, 1, 1))])
def test_conv_kernel_geometry(executor, k, s, pads):
    check(K.conv_case(100 + k[0] * 13 + s[0], 2, 23, 19, 32, 32, k=k, s=s, pads=pads), executor)


@pytest.mark.parametrize("in_signed,w_signed,in_zp,w_zp,out_signed,out_zp", [
    (False, True, 128, 0, False, 128),   # the benchmark types
    (False, True, 0, 0, False, 0),
    (False, True, 3, 0, False, 17),      # zero point away from the storage offset: weight-sum correction
    (True, True, 0, 0, True, 0),
    (True, True, -7, 0, True, -128),
    (False, False, 128, 128, False, 128),
    (False, False, 121, 127, False, 255),  # both corrections
    (True, False, 5, 3, False, 9),
])
def test_conv_types_and_zero_points(executor, in_signed, w_signed, in_zp, w_zp, out_signed, out_zp):
    check(K.conv_case(7, 1, 10, 10, 32, 32, in_signed=in_signed, w_signed=w_signed, in_zp=in_zp, w_zp=w_zp,
                      out_signed=out_signed, out_zp=out_zp), executor)


PPE_VARIANTS = [
    dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255),
    dict(mode=nce.PPE_NOOP, clamp_low=128, clamp_high=255),                              # ReLU the 37XX way
    dict(mode=nce.PPE_LRELU, clamp_low=0, clamp_high=255),
    dict(mode=nce.PPE_LRELUX, clamp_low=0, clamp_high=200),
    dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14),
    dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=-5, lrelu_shift=2),
    dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=2047, lrelu_shift=31),
    dict(mode=nce.PPE_NOOP, clamp_low=-128, clamp_high=127, clamp_domain=nce.CLAMP_PRE_ZP),
    dict(mode=nce.PPE_LRELU, clamp_low=0, clamp_high=100, clamp_domain=nce.CLAMP_PRE_ZP),
    dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255, round_mode=nce.ROUND_HALF_EVEN),
    dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=3, lrelu_shift=1, round_mode=nce.ROUND_HALF_EVEN),
    dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255, round_mode=nce.ROUND_NONE),
    {},                                                                                 # no PPE task at all
]


@pytest.mark.parametrize("ppe", PPE_VARIANTS)
def test_conv_ppe_variants(executor, ppe):
    check(K.conv_case(21, 1, 12, 12, 32, 32, ppe=ppe), executor)


@pytest.mark.parametrize("scale_lo,scale_hi", [(1e-6, 1e-5), (1e-2, 1e-1), (0.3, 0.9), (1.0, 7.9), (20.0, 255.0),
                                               (2e-13, 9e-13), (1e-12, 1e-3)])
def test_conv_scale_ranges(executor, scale_lo, scale_hi):
    # small scales -> shift up to 34; large scales -> shift down to 7 and saturating outputs
    check(K.conv_case(33, 1, 8, 8, 32, 32, scale_lo=scale_lo, scale_hi=scale_hi), executor)


@pytest.mark.parametrize("scale_lo,scale_hi", [(2e-13, 9e-13), (1e-12, 1e-3), (3.0, 200.0)])
def test_dwconv_scale_ranges(executor, scale_lo, scale_hi):
    # shifts above 52 take the integer epilogue, shifts below 18 the saturating one
    check(K.dw_case(34, 1, 9, 9, 32, scale_lo=scale_lo, scale_hi=scale_hi), executor)
    check(K.dw_case(35, 1, 9, 9, 32, scale_lo=scale_lo, scale_hi=scale_hi,
                    ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=2047, lrelu_shift=0)), executor)


def test_dwconv_cfg3_small(executor):
    check(K.cfg3_dw(n=1), executor)


@pytest.mark.parametrize("c,k,s,pads", [(16, (3, 3), (1, 1), (1, 1, 1, 1)), (96, (3, 3), (2, 2), (1, 1, 1, 1)),
                                        (272, (5, 5), (1, 1), (2, 2, 2, 2)), (32, (11, 11), (3, 3), (5, 5, 5, 5)),
                                        (48, (2, 3), (2, 1), (1, 1, 0, 1)), (512, (3, 3), (2, 2), (0, 0, 0, 0))])
def test_dwconv_shapes(executor, c, k, s, pads):
    check(K.dw_case(5 + c, 2, 21, 17, c, k=k, s=s, pads=pads), executor)


@pytest.mark.parametrize("in_signed,w_signed,in_zp,w_zp", [(False, False, 100, 131), (True, True, -3, 0), (True, False, 1, 2)])
def test_dwconv_types(executor, in_signed, w_signed, in_zp, w_zp):
    check(K.dw_case(9, 1, 12, 12, 32, in_signed=in_signed, w_signed=w_signed, in_zp=in_zp, w_zp=w_zp,
                    out_signed=in_signed, out_zp=-5 if in_signed else 77), executor)


@pytest.mark.parametrize("is_max", [True, False])
@pytest.mark.parametrize("k,s,pads", [((3, 3), (2, 2), (1, 1, 1, 1)), ((2, 2), (2, 2), (0, 0, 0, 0)),
                                      ((3, 3), (1, 1), (1, 1, 1, 1)), ((7, 7), (7, 7), (0, 0, 0, 0))])
def test_pools(executor, is_max, k, s, pads):
    check(K.pool_case(3, is_max, 2, 28, 28, 96, k=k, s=s, pads=pads), executor)
    check(K.pool_case(4, is_max, 1, 14, 14, 32, k=k, s=s, pads=pads, in_signed=True, in_zp=-11, out_zp=4), executor)


def test_avgpool_with_weight_table(executor):
    check(K.pool_case(6, False, 2, 14, 14, 64, with_table=True), executor)


@pytest.mark.parametrize("out_signed,lo,hi", [(True, -300, 300), (True, -128, 127), (True, -100, 90), (False, -40, 300), (False, 7, 200)])
def test_window_clamp_bounds(executor, out_signed, lo, hi):
    """Depthwise and average pool with clamp bounds inside and outside the storage range, signed and unsigned outputs
    (the kernels choose between a truncating and a flooring conversion from the lower bound)."""
    ppe = dict(mode=nce.PPE_NOOP, clamp_low=lo, clamp_high=hi)
    check(K.dw_case(71, 2, 40, 36, 96, out_signed=out_signed, out_zp=-9 if out_signed else 131, ppe=ppe), executor)
    m, sh = K.approx(15, 1.0 / 9)
    check(K.pool_case(72, False, 2, 40, 36, 96, in_signed=out_signed, in_zp=-4 if out_signed else 120, out_zp=-9 if out_signed else 131,
                      ppe=dict(ppe, quant_mult=m, quant_shift=sh)), executor)


def test_window_strided_input_view(executor):
    """Depthwise over an input that is a sub-view of a larger tensor (W, H and N strides larger than the compact ones):
    interior wavefronts address their taps as 32-bit offsets into the view."""
    import torch
    case = K.dw_case(73, 2, 40, 36, 64, s=(1, 1))
    want = K.run_oracle(case)
    big_in = torch.zeros((2, 44, 40, 96), dtype=torch.uint8, device="cuda")
    view_in = big_in[:, 3:43, 2:38, 16:80]
    view_in.copy_(torch.from_numpy(case.input).cuda())
    out = torch.zeros(case.out_shape, dtype=torch.uint8, device="cuda")
    w = torch.from_numpy(case.weights).cuda()
    t = torch.from_numpy(case.table).cuda()
    task = K.build_task(case, view_in, w, t, out)
    stream = torch.cuda.current_stream().cuda_stream
    executor.enqueue(task, stream)
    executor.synchronize(stream)
    assert np.array_equal(out.cpu().numpy(), want)


def test_maxpool_clamped(executor):
    check(K.pool_case(8, True, 1, 14, 14, 32, ppe=dict(mode=nce.PPE_NOOP, clamp_low=30, clamp_high=200)), executor)


def test_eltwise_cfg4_small(executor):
    check(K.cfg4(n=2), executor)


@pytest.mark.parametrize("kw", [dict(with_in_mult=False, mult=16384, shift=15),
                                dict(signed=True, zp_a=-3, zp_b=12, out_zp=-100),
                                dict(with_table=True),
                                dict(ppe_extra=dict(round_mode=nce.ROUND_HALF_EVEN)),
                                dict(ppe_extra=dict(mode=nce.PPE_LRELU, clamp_low=128)),
                                dict(in1_mult=65535, in2_mult=65535, mult=65535, shift=40),
                                dict(mult=3, shift=0, in1_mult=1, in2_mult=1),
                                dict(mult=40000, shift=53), dict(mult=65535, shift=63),
                                dict(mult=65535, shift=10, ppe_extra=dict(mode=nce.PPE_LPRELU, lrelu_mult=-2047, lrelu_shift=0)),
                                dict(ppe_extra=dict(round_mode=nce.ROUND_NONE))])
def test_eltwise_variants(executor, kw):
    check(K.eltwise_case(11, 1, 7, 9, 48, **kw), executor)


# ---- variants: any tiling of the output box gives the same bytes ---------------------------------

@pytest.mark.parametrize("onto", [1, 2])
@pytest.mark.parametrize("variants", [False, True])
def test_eltwise_in_place(executor, onto, variants):
    """An eltwise flagged is_inplace writes its output over its first (second) input; the bytes are those of the same
    add into a separate tensor."""
    import torch
    case = K.eltwise_case(91, 2, 9, 13, 48, signed=True, zp_a=-3, zp_b=12, out_zp=-100) if onto == 2 else K.eltwise_case(91, 2, 9, 13, 48)
    if variants:
        case.variants = [((0, 0, 0), (12, 3, 47)), ((0, 4, 0), (12, 8, 15)), ((0, 4, 16), (12, 8, 47))]
    print(f"[case] eltwise in place onto input {onto}, variants={variants}", flush=True)
    want = K.run_oracle(case)
    a = torch.from_numpy(case.input).to("cuda:0")
    b = torch.from_numpy(case.weights).to("cuda:0")
    out = a if onto == 1 else b
    task = K.build_task(case, a, b, None, out)
    task.desc.flags = 1 << 4
    stream = torch.cuda.current_stream().cuda_stream
    executor.enqueue(task, stream)
    executor.synchronize(stream)
    assert np.array_equal(out.cpu().numpy(), want)
    other = b if onto == 1 else a
    assert np.array_equal(other.cpu().numpy(), case.weights if onto == 1 else case.input), "the other input was touched"


def _tilings(oh, ow, oc):
    yield [((0, 0, 0), (ow - 1, oh // 2 - 1, oc - 1)), ((0, oh // 2, 0), (ow - 1, oh - 1, oc - 1))]       # split over height
    yield [((0, 0, 0), (ow - 1, oh - 1, 15)), ((0, 0, 16), (ow - 1, oh - 1, oc - 1))]                     # split over channels
    yield [((0, 0, 0), (ow // 3, oh - 1, oc - 1)), ((ow // 3 + 1, 0, 0), (ow - 1, oh - 1, oc - 1))]       # split over width
    yield [((1, 2, 16), (ow - 2, oh - 2, oc - 1))]                                                       # partial cover


@pytest.mark.parametrize("which", range(4))
def test_variant_tilings(executor, which):
    for maker in (lambda v: K.conv_case(41, 2, 12, 10, 32, 48, variants=v),
                  lambda v: K.dw_case(42, 2, 24, 20, 48, variants=v),
                  lambda v: K.pool_case(43, True, 2, 24, 20, 48, variants=v),
                  lambda v: K.pool_case(44, False, 2, 24, 20, 48, variants=v),
                  lambda v: K.eltwise_case(45, 2, 12, 10, 48, variants=v)):
        probe = maker(None)
        _, oh, ow, oc = probe.out_shape
        tiling = list(_tilings(oh, ow, oc))[which]
        case = maker(tiling)
        # bytes outside the variants must stay untouched: compare against the oracle run on the same
        # poisoned canvas
        want = np.full(case.out_shape, 0x5A, dtype=np.uint8)
        from oracle import nce_oracle
        nce_oracle.run(K.build_task(case, case.input, case.weights, case.table, want))
        got = K.run_hip(case, executor)
        assert np.array_equal(want, got), f"{case.name} tiling {which}"
        if which < 3:
            assert np.array_equal(got, K.run_oracle(probe)), "a full tiling must equal the single-variant result"


def test_strided_views(executor):
    """parent_input / parent_output style sub-views: W and H strides larger than the compact ones."""
    import torch
    case = K.conv_case(51, 1, 8, 8, 32, 32)
    want = K.run_oracle(case)
    big_in = torch.zeros((1, 10, 12, 64), dtype=torch.uint8, device="cuda")
    big_out = torch.zeros((1, 9, 11, 48), dtype=torch.uint8, device="cuda")
    view_in = big_in[:, 1:9, 2:10, 16:48]
    view_in.copy_(torch.from_numpy(case.input).cuda())
    view_out = big_out[:, 0:8, 1:9, 16:48]
    w = torch.from_numpy(case.weights).cuda()
    t = torch.from_numpy(case.table).cuda()
    task = K.build_task(case, view_in, w, t, view_out)
    stream = torch.cuda.current_stream().cuda_stream
    executor.enqueue(task, stream)
    executor.synchronize(stream)
    assert np.array_equal(view_out.cpu().numpy(), want)
    mask = torch.ones_like(big_out, dtype=torch.bool)
    mask[:, 0:8, 1:9, 16:48] = False
    assert not big_out[mask].any(), "bytes outside the output view were written"


def test_determinism(executor):
    case = K.cfg2(n=1)
    first = K.run_hip(case, executor)
    for _ in range(3):
        assert np.array_equal(first, K.run_hip(case, executor))


def test_task_list_chain(executor):
    """conv -> maxpool -> eltwise(add with itself) chained through a task list on one stream."""
    import torch
    c1 = K.conv_case(61, 2, 16, 16, 32, 32)
    y1 = K.run_oracle(c1)
    c2 = K.pool_case(62, True, 2, 16, 16, 32)
    c2.input = y1
    y2 = K.run_oracle(c2)
    c3 = K.eltwise_case(63, 2, 8, 8, 32)
    c3.input = y2
    c3.weights = y2
    y3 = K.run_oracle(c3)

    d1 = K.DeviceCase(c1)
    d2 = K.DeviceCase(c2)
    d3 = K.DeviceCase(c3)
    t2 = K.build_task(c2, d1.output, None, None, d2.output)
    t3 = K.build_task(c3, d2.output, d2.output, None, d3.output)
    tl = executor.task_list()
    for t in (d1.task, t2, t3):
        tl.append(t)
    stream = torch.cuda.current_stream().cuda_stream
    tl.enqueue(stream)
    executor.synchronize(stream)
    tl.destroy()
    assert np.array_equal(d3.output.cpu().numpy(), y3)


# ---- cfg5: the ResNet-50 task graph ---------------------------------------------------------------

@pytest.mark.parametrize("batch,size", [(3, 96)])
def test_resnet50_graph_every_tensor(executor, batch, size):
    """All 70 tasks (53 convs, max pool, 16 adds) chained on the GPU through one task list; every
    intermediate tensor must equal the oracle's, not just the last one."""
    import torch
    graph = K.ResNet50Graph(batch=batch, size=size)
    x = graph.make_input()
    print(f"[case] resnet50 graph batch={batch} size={size}", flush=True)
    want = K.run_graph_oracle(graph, x)
    dg = K.DeviceGraph(graph, executor, x)
    stream = torch.cuda.current_stream().cuda_stream
    dg.run(stream)
    executor.synchronize(stream)
    for L in graph.layers:
        got = dg.buffers[L.dst].cpu().numpy()
        assert np.array_equal(got, want[L.dst]), f"{L.name}: {(got != want[L.dst]).sum()} bytes differ"
    assert len(np.unique(want[graph.output])) > 100, "degenerate network output"
    dg.task_list.destroy()


# ---- weights-resident conv kernel: every instantiation (channel fragments x pixel fragments x path) ---

WRES_CONFIGS = ["4,4,8,1", "4,2,8,2", "4,1,4,1", "2,4,8,1", "2,2,4,3", "2,1,8,1"]  # nf, bf, waves, tiles per wave
WRES_SHAPES = [
    # (n, h, w, ic, oc, k, s, pads, in_zp)
    (2, 20, 20, 64, 64, (1, 1), (1, 1), (0, 0, 0, 0), 128),    # one reduction step (padded to two), no masks
    (2, 20, 20, 256, 80, (1, 1), (1, 1), (0, 0, 0, 0), 5),     # four steps (deep ring), weight sums, ragged channels
    (3, 19, 17, 64, 48, (3, 3), (1, 1), (1, 1, 1, 1), 128),    # tap masks, odd step count, partial pixel tile
    (2, 21, 21, 128, 64, (3, 3), (2, 2), (1, 1, 1, 1), 200),   # stride 2 with masks and weight sums
    (2, 30, 30, 16, 64, (7, 7), (2, 2), (3, 3, 3, 3), 114),    # per-lane tap path: 16 channels, 49 taps
    (2, 12, 12, 48, 32, (3, 3), (1, 1), (1, 1, 1, 1), 77),     # per-lane tap path: steps straddle taps
    (1, 9, 9, 64, 16, (3, 3), (1, 1), (0, 0, 0, 0), 128),      # 3x3 without padding: every tap inside
    (2, 10, 10, 192, 144, (1, 1), (2, 2), (0, 0, 0, 0), 0),    # 1x1 stride 2, three steps padded to four
    (1, 12, 12, 128, 48, (3, 3), (1, 1), (0, 0, 0, 0), 128),   # permuted activation loads, every tap inside, ragged channels
    (2, 9, 9, 192, 64, (3, 3), (1, 1), (1, 1, 1, 1), 99),      # permuted loads with tap masks, 27 steps (depth 3)
    (1, 5, 7, 2048, 48, (1, 1), (1, 1), (0, 0, 0, 0), 17),     # permuted loads on a long dense 1x1 reduction, partial tile
]


@pytest.mark.parametrize("config", WRES_CONFIGS)
@pytest.mark.parametrize("shape", WRES_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}s{s[6][0]}")
def test_conv_weights_resident_instantiations(tuned, shape, config):
    n, h, w, ic, oc, k, s, pads, in_zp = shape
    executor = tuned(NCE_HIP_CONV_WRES=config)
    check(K.conv_case(400 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=in_zp, out_zp=9,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=250, lrelu_mult=1638, lrelu_shift=14)), executor)


@pytest.mark.parametrize("config", ["4,2,8,1", "2,1,4,2"])
def test_conv_weights_resident_types_and_modes(tuned, config):
    executor = tuned(NCE_HIP_CONV_WRES=config)
    check(K.conv_case(421, 2, 14, 14, 64, 64, in_signed=True, in_zp=-7, out_signed=True, out_zp=-128), executor)
    check(K.conv_case(422, 2, 14, 14, 64, 64, w_signed=False, w_zp=128, in_zp=121), executor)
    check(K.conv_case(423, 2, 14, 14, 64, 64, in_zp=3, ppe=dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255,
                                                                 round_mode=nce.ROUND_HALF_EVEN)), executor)   # integer PPE path
    check(K.conv_case(424, 2, 14, 14, 64, 64, in_zp=3, scale_lo=20.0, scale_hi=255.0), executor)               # may saturate int32
    check(K.conv_case(425, 2, 14, 14, 64, 64, in_zp=250, ppe=dict(mode=nce.PPE_NOOP, clamp_low=128, clamp_high=255)), executor)
    # the same with pixels 128 bytes apart and a 3x3 kernel: activation loads in pixel-major lane order
    wide = dict(k=(3, 3), pads=(1, 1, 1, 1))
    check(K.conv_case(426, 2, 11, 11, 128, 64, in_signed=True, in_zp=-7, out_signed=True, out_zp=-128, **wide), executor)
    check(K.conv_case(427, 2, 11, 11, 128, 64, w_signed=False, w_zp=128, in_zp=121, **wide), executor)
    check(K.conv_case(428, 2, 11, 11, 128, 64, in_zp=3, ppe=dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255,
                                                                 round_mode=nce.ROUND_HALF_EVEN), **wide), executor)
    check(K.conv_case(429, 2, 11, 11, 128, 64, in_zp=3, scale_lo=20.0, scale_hi=255.0, **wide), executor)
    check(K.conv_case(430, 2, 11, 11, 128, 64, in_zp=250, ppe=dict(mode=nce.PPE_NOOP, clamp_low=128, clamp_high=255), **wide), executor)


WZP_SHAPES = [
    # (n, h, w, ic, oc, k, s, pads): weights whose zero point is not their storage offset
    (2, 20, 20, 64, 64, (1, 1), (1, 1), (0, 0, 0, 0)),     # one step, padded to two: the padding step must read the fill line
    (3, 19, 17, 64, 48, (3, 3), (1, 1), (1, 1, 1, 1)),     # nine steps (padded to ten), tap masks, partial tile
    (1, 9, 9, 64, 16, (3, 3), (1, 1), (0, 0, 0, 0)),       # no padding of the image, odd step count: mask mode forced
    (2, 21, 21, 128, 64, (3, 3), (2, 2), (1, 1, 1, 1)),    # permuted loads, 18 steps
    (1, 12, 12, 256, 48, (3, 3), (1, 1), (0, 0, 0, 0)),    # permuted loads, depth 4, ragged channels
    (2, 12, 12, 48, 32, (3, 3), (1, 1), (1, 1, 1, 1)),     # per-lane tap path
    (2, 10, 10, 192, 144, (1, 1), (2, 2), (0, 0, 0, 0)),   # 1x1 stride 2, three steps padded to four
]


@pytest.mark.parametrize("config", ["4,4,8,1", "4,2,8,2", "4,1,4,1", "2,2,4,3", "2,1,8,1"])
@pytest.mark.parametrize("shape", WZP_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}s{s[6][0]}")
def test_conv_weights_resident_weight_zero_point(tuned, shape, config):
    n, h, w, ic, oc, k, s, pads = shape
    executor = tuned(NCE_HIP_CONV_WRES=config)
    # u8 weights around 117 (offset +11 from the re-biased storage), then i8 weights with zero point 5
    check(K.conv_case(600 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=131, w_signed=False, w_zp=117, out_zp=9,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=250, lrelu_mult=1638, lrelu_shift=14)), executor)
    check(K.conv_case(700 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_signed=True, in_zp=-3, w_signed=True, w_zp=5), executor)


def test_conv_weights_resident_variants(tuned):
    executor = tuned(NCE_HIP_CONV_WRES="2,2,4,1")
    test_conv_halo_variants(executor)
    test_conv_halo_variants(executor, ic=128)   # permuted activation loads, boxes that start inside the image


# ---- halo-staged conv kernel: every tile configuration, image-crossing tiles, partial slices -----
# (the dispatcher prefers the weights-resident kernel; NCE_HIP_CONV_PATH=1 sends these to the halo kernel)

@pytest.fixture
def halo_path(tuned):
    return tuned(NCE_HIP_CONV_PATH="1")


@pytest.fixture
def gather_path(tuned):
    return tuned(NCE_HIP_CONV_PATH="2")


HALO_CASES = [
    # (n, h, w, ic, oc, k, s, pads)                      which tile the dispatcher picks
    (8, 128, 128, 64, 128, (3, 3), (1, 1), (1, 1, 1, 1)),   # 128 ch x 256 px
    (4, 128, 128, 64, 128, (3, 3), (1, 1), (1, 1, 1, 1)),   # 64 ch x 256 px
    (1, 128, 128, 64, 128, (3, 3), (1, 1), (1, 1, 1, 1)),   # 64 ch x 128 px
    (8, 56, 56, 64, 64, (3, 3), (1, 1), (1, 1, 1, 1)),      # 64 ch x 64 px (cfg2 shape)
    (8, 128, 128, 128, 256, (1, 1), (1, 1), (0, 0, 0, 0)),  # 1x1, big tile
    (2, 56, 56, 256, 64, (1, 1), (1, 1), (0, 0, 0, 0)),     # 1x1, deep K
    (2, 56, 56, 256, 512, (1, 1), (2, 2), (0, 0, 0, 0)),    # 1x1 stride 2 (downsample)
    (3, 56, 56, 128, 128, (3, 3), (2, 2), (1, 1, 1, 1)),    # 3x3 stride 2
    (40, 7, 7, 512, 128, (3, 3), (1, 1), (1, 1, 1, 1)),     # tiles span several whole images
    (9, 14, 14, 256, 256, (3, 3), (1, 1), (1, 1, 1, 1)),    # tiles cross image boundaries mid-row
    (2, 30, 30, 96, 80, (3, 3), (1, 1), (1, 1, 1, 1)),      # partial 64-channel slice, ragged channels
    (2, 30, 30, 160, 48, (1, 1), (1, 1), (0, 0, 0, 0)),
    (2, 31, 29, 64, 64, (3, 3), (1, 2), (0, 1, 1, 0)),      # asymmetric stride and padding
    (2, 20, 20, 64, 64, (5, 3), (1, 1), (1, 1, 2, 2)),      # tall kernel
    (2, 20, 20, 64, 64, (1, 3), (1, 1), (1, 1, 0, 0)),
]


@pytest.mark.parametrize("shape", HALO_CASES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}x{s[5][1]}s{s[6][0]}")
def test_conv_halo_kernel_shapes(halo_path, shape):
    executor = halo_path
    n, h, w, ic, oc, k, s, pads = shape
    check(K.conv_case(200 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14)), executor)


def test_conv_halo_zero_points_and_types(halo_path):
    executor = halo_path
    check(K.conv_case(301, 2, 20, 20, 64, 64, in_zp=3, out_zp=17), executor)                      # weight-sum correction
    check(K.conv_case(302, 2, 20, 20, 128, 64, in_signed=True, in_zp=-7, out_signed=True, out_zp=-128), executor)
    check(K.conv_case(303, 2, 20, 20, 64, 64, w_signed=False, w_zp=128, in_zp=121), executor)
    check(K.conv_case(304, 2, 20, 20, 64, 64, w_signed=False, w_zp=127, in_zp=121), executor)      # falls back to the gather kernel


def test_conv_halo_variants(executor, ic=64):
    full = K.conv_case(305, 2, 24, 20, ic, 128)
    want = K.run_oracle(full)
    tiled = K.conv_case(305, 2, 24, 20, ic, 128, variants=[((0, 0, 0), (19, 11, 63)), ((0, 12, 0), (19, 23, 63)),
                                                           ((0, 0, 64), (9, 23, 127)), ((10, 0, 64), (19, 23, 127))])
    assert np.array_equal(K.run_hip(tiled, executor), want)
    part = K.conv_case(305, 2, 24, 20, ic, 128, variants=[((3, 5, 64), (17, 20, 127))])
    canvas = np.full(part.out_shape, 0x5A, dtype=np.uint8)
    from oracle import nce_oracle
    nce_oracle.run(K.build_task(part, part.input, part.weights, part.table, canvas))
    assert np.array_equal(K.run_hip(part, executor), canvas)


def test_conv_halo_variants_on_halo_path(halo_path):
    test_conv_halo_variants(halo_path)


@pytest.mark.parametrize("shape", [HALO_CASES[3], HALO_CASES[6], HALO_CASES[10], HALO_CASES[12]],
                         ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}x{s[5][1]}s{s[6][0]}")
def test_conv_gather_kernel_shapes(gather_path, shape):
    executor = gather_path
    n, h, w, ic, oc, k, s, pads = shape
    check(K.conv_case(500 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=77,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14)), executor)


def test_conv_wide_kernel_falls_back(executor):
    # 7x7 with 64 input channels needs more than 31 tap bits: the halo / gather kernels take it
    check(K.conv_case(511, 1, 20, 20, 64, 32, k=(7, 7), s=(1, 1), pads=(3, 3, 3, 3), in_zp=100), executor)


# ---- ODU permutation: outputs written in any order of H, W, C ----------------------------------------

ODU_ORDERS = {"nhwc": (0, 1, 2, 3), "nwhc": (0, 2, 1, 3), "nwch": (0, 2, 3, 1), "ncwh": (0, 3, 2, 1),
              "nhcw": (0, 1, 3, 2), "nchw": (0, 3, 1, 2)}   # memory order as axes of the (N, H, W, C) result


def _permuted_run(case, order, executor):
    """Runs the case with its output laid out in `order`; returns (hip, oracle) as (N, H, W, C) arrays."""
    import torch
    from oracle import nce_oracle
    axes = ODU_ORDERS[order]
    inverse = [axes.index(i) for i in range(4)]
    mem_shape = tuple(case.out_shape[a] for a in axes)
    host = np.full(mem_shape, 0x5A, dtype=np.uint8)
    nce_oracle.run(K.build_task(case, case.input, case.weights, case.table, host.transpose(inverse)))
    dc = K.DeviceCase(case)
    dev = torch.full(mem_shape, 0x5A, dtype=torch.uint8, device="cuda")
    task = K.build_task(case, dc.input, dc.weights, dc.table, dev.permute(*inverse))
    stream = torch.cuda.current_stream().cuda_stream
    executor.enqueue(task, stream)
    executor.synchronize(stream)
    return dev.cpu().numpy().transpose(inverse), host.transpose(inverse)


@pytest.mark.parametrize("order", list(ODU_ORDERS))
def test_odu_permutation_conv(executor, order):
    case = K.conv_case(600, 2, 11, 13, 64, 48, in_zp=99,
                       ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14))
    got, want = _permuted_run(case, order, executor)
    assert np.array_equal(want, K.run_oracle(case)), "the oracle itself must be layout-independent"
    assert np.array_equal(got, want)


@pytest.mark.parametrize("order", ["nchw", "nwch", "nhcw"])
def test_odu_permutation_other_tasks(executor, order, tuned):
    cases = [K.conv_case(601, 1, 9, 9, 16, 32, k=(5, 5), pads=(2, 2, 2, 2)),            # per-lane tap path
             K.dw_case(602, 2, 13, 13, 32), K.pool_case(603, True, 2, 12, 12, 32), K.pool_case(604, False, 2, 12, 12, 32),
             K.eltwise_case(605, 2, 9, 7, 48)]
    for case in cases:
        got, want = _permuted_run(case, order, executor)
        assert np.array_equal(got, want), case.name
    for path in ("1", "2"):  # halo and gather kernels
        got, want = _permuted_run(K.conv_case(606, 2, 10, 10, 64, 64), order, tuned(NCE_HIP_CONV_PATH=path))
        assert np.array_equal(got, want), f"conv path {path}"


def test_odu_permutation_variants_leave_other_bytes_alone(executor):
    case = K.conv_case(607, 1, 12, 12, 64, 64, variants=[((2, 3, 16), (9, 10, 47))])
    got, want = _permuted_run(case, "nchw", executor)
    assert np.array_equal(got, want) and (want == 0x5A).sum() > want.size // 2


# ---- reductions longer than one LDS slice: weights staged chunk by chunk ------------------------------

LONG_K_SHAPES = [
    # (n, h, w, ic, oc, k, s, pads)
    (1, 6, 6, 1024, 48, (3, 3), (1, 1), (1, 1, 1, 1)),     # 9216 bytes: two chunks, tap masks, ragged channels
    (2, 7, 5, 256, 32, (5, 5), (1, 1), (2, 2, 2, 2)),      # 6400 bytes, 25 taps
    (1, 9, 9, 128, 64, (7, 7), (2, 2), (3, 3, 3, 3)),      # 49 taps (more than the tap-mask kernels take), stride 2
    (1, 5, 7, 8192, 32, (1, 1), (1, 1), (0, 0, 0, 0)),     # 1x1 over 8192 channels: two chunks, partial tile
    (1, 4, 4, 4672, 32, (1, 1), (1, 1), (0, 0, 0, 0)),     # 73 steps: padded to 76, second chunk of four steps
]


@pytest.mark.parametrize("config", ["2,1,8,1", "2,2,4,1", "2,1,3,1"])
@pytest.mark.parametrize("shape", LONG_K_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}s{s[6][0]}")
def test_conv_long_reduction(tuned, shape, config):
    n, h, w, ic, oc, k, s, pads = shape
    executor = tuned(NCE_HIP_CONV_WRES=config)
    check(K.conv_case(800 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=119, out_zp=3,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=250, lrelu_mult=1638, lrelu_shift=14)), executor)
    # weights whose zero point is not their storage offset
    check(K.conv_case(900 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=119, w_signed=False, w_zp=140), executor)


def test_conv_wide_padded_kernel_on_chunked_kernel(executor):
    # 7x7 with padding over 64 channels fits LDS but needs more than 31 tap bits: row / column bits of the chunked kernel
    check(K.conv_case(512, 2, 13, 11, 64, 48, k=(7, 7), s=(1, 1), pads=(3, 3, 3, 3), in_zp=100), executor)
    check(K.conv_case(513, 1, 13, 11, 128, 32, k=(6, 6), s=(2, 2), pads=(2, 2, 3, 3), in_zp=7, w_signed=False, w_zp=131), executor)


# ---- seeded random convolutions: kernel variants are picked by shape, so sweep shapes ---------------------------------

def _random_conv_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        ky, kx = (int(rng.integers(1, 6)), int(rng.integers(1, 6))) if rng.random() < 0.3 else (int(rng.choice([1, 3, 3, 5, 7])),) * 2
        sy, sx = (int(rng.integers(1, 3)),) * 2 if rng.random() < 0.7 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        ic = int(rng.choice([16, 32, 48, 64, 64, 96, 128, 128, 192, 256, 320, 512]))
        oc = int(rng.choice([16, 32, 48, 64, 80, 128, 144]))
        pads = (int(rng.integers(0, kx // 2 + 1)), int(rng.integers(0, kx // 2 + 1)),   # left, right
                int(rng.integers(0, ky // 2 + 1)), int(rng.integers(0, ky // 2 + 1)))   # top, bottom
        h = int(rng.integers(max(ky, 3), 15))
        w = int(rng.integers(max(kx, 3), 15))
        n = int(rng.integers(1, 4))
        in_signed = bool(rng.random() < 0.3)
        w_signed = bool(rng.random() < 0.7)
        in_zp = int(rng.integers(-128, 128)) if in_signed else int(rng.integers(0, 256))
        w_zp = (0 if rng.random() < 0.6 else int(rng.integers(-20, 20))) if w_signed else (128 if rng.random() < 0.5 else int(rng.integers(100, 156)))
        out_signed = bool(rng.random() < 0.3)
        out_zp = int(rng.integers(-100, 100)) if out_signed else int(rng.integers(0, 200))
        lo, hi = (-128, 127) if out_signed else (0, 255)   # clamp bounds in the output domain (after the zero point)
        mode = rng.choice(["noop", "relu", "lrelu"])
        if mode == "noop":
            ppe = dict(mode=nce.PPE_NOOP, clamp_low=lo, clamp_high=hi)
        elif mode == "relu":
            ppe = dict(mode=nce.PPE_LRELU, clamp_low=max(lo, out_zp), clamp_high=hi)
        else:
            ppe = dict(mode=nce.PPE_LPRELU, clamp_low=lo, clamp_high=int(rng.integers(out_zp + 1, hi + 1)),
                       lrelu_mult=int(rng.integers(1, 2048)), lrelu_shift=int(rng.integers(11, 16)))
        cases.append(dict(seed=1000 + i, n=n, h=h, w=w, ic=ic, oc=oc, k=(ky, kx), s=(sy, sx), pads=pads,
                          in_signed=in_signed, w_signed=w_signed, in_zp=in_zp, w_zp=w_zp, out_signed=out_signed, out_zp=out_zp, ppe=ppe))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(128, 20251), ids=lambda c: f"{c['n']}x{c['h']}x{c['w']}x{c['ic']}_{c['oc']}_k{c['k'][0]}x{c['k'][1]}s{c['s'][0]}x{c['s'][1]}")
def test_conv_random_shapes(executor, case):
    c = dict(case)
    seed, n, h, w, ic, oc = (c.pop(k) for k in ("seed", "n", "h", "w", "ic", "oc"))
    left, right, top, bottom = c["pads"]
    if (h + top + bottom - c["k"][0]) // c["s"][0] + 1 < 1 or (w + left + right - c["k"][1]) // c["s"][1] + 1 < 1:
        pytest.skip("window larger than the padded image")
    check(K.conv_case(seed, n, h, w, ic, oc, **c), executor)


def _random_window_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        kind = str(rng.choice(["dw", "max", "avg"]))
        ky, kx = (int(rng.integers(1, 6)), int(rng.integers(1, 6))) if rng.random() < 0.4 else (int(rng.choice([2, 3, 3, 5])),) * 2
        sy, sx = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pads = (int(rng.integers(0, kx // 2 + 1)), int(rng.integers(0, kx // 2 + 1)),
                int(rng.integers(0, ky // 2 + 1)), int(rng.integers(0, ky // 2 + 1)))
        c = 16 * int(rng.integers(1, 20))
        h = int(rng.integers(max(ky, 3), 20))
        w = int(rng.integers(max(kx, 3), 20))
        n = int(rng.integers(1, 4))
        in_signed = bool(rng.random() < 0.4)
        in_zp = int(rng.integers(-128, 128)) if in_signed else int(rng.integers(0, 256))
        cases.append(dict(kind=kind, seed=2000 + i, n=n, h=h, w=w, c=c, k=(ky, kx), s=(sy, sx), pads=pads, in_signed=in_signed, in_zp=in_zp,
                          w_signed=bool(rng.random() < 0.6), w_zp=int(rng.integers(-10, 10)), with_table=bool(rng.random() < 0.5)))
    return cases


@pytest.mark.parametrize("case", _random_window_cases(64, 777), ids=lambda c: f"{c['kind']}_{c['n']}x{c['h']}x{c['w']}x{c['c']}_k{c['k'][0]}x{c['k'][1]}s{c['s'][0]}x{c['s'][1]}")
def test_window_random_shapes(executor, case):
    c = dict(case)
    kind, seed, n, h, w, ch = (c.pop(k) for k in ("kind", "seed", "n", "h", "w", "c"))
    w_signed, w_zp, with_table = c.pop("w_signed"), c.pop("w_zp"), c.pop("with_table")
    if kind == "dw":
        zp = w_zp if w_signed else 128 + w_zp
        check(K.dw_case(seed, n, h, w, ch, w_signed=w_signed, w_zp=zp, **c), executor)
    else:
        out_zp = 0 if kind == "max" else (c["in_zp"] // 2 if c["in_signed"] else 128 + c["in_zp"] // 4)
        check(K.pool_case(seed, kind == "max", n, h, w, ch, with_table=with_table, out_zp=out_zp, **c), executor)


def _random_eltwise_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        signed = bool(rng.random() < 0.4)
        zp = (lambda: int(rng.integers(-128, 128))) if signed else (lambda: int(rng.integers(0, 256)))
        mult = int(rng.integers(8192, 65536))
        shift = int(rng.integers(18, 36))
        extra = {}
        if rng.random() < 0.3:
            extra = dict(mode=nce.PPE_LPRELU, lrelu_mult=int(rng.integers(1, 2048)), lrelu_shift=int(rng.integers(11, 16)))
        cases.append(dict(seed=3000 + i, n=int(rng.integers(1, 4)), h=int(rng.integers(1, 17)), w=int(rng.integers(1, 17)),
                          c=16 * int(rng.integers(1, 24)), signed=signed, zp_a=zp(), zp_b=zp(), out_zp=zp(),
                          in1_mult=int(rng.integers(1, 65536)), in2_mult=int(rng.integers(1, 65536)), mult=mult, shift=shift,
                          with_in_mult=bool(rng.random() < 0.8), with_table=bool(rng.random() < 0.25), ppe_extra=extra or None))
    return cases


@pytest.mark.parametrize("case", _random_eltwise_cases(48, 4242), ids=lambda c: f"{c['n']}x{c['h']}x{c['w']}x{c['c']}_{'i8' if c['signed'] else 'u8'}_s{c['shift']}")
def test_eltwise_random(executor, case):
    c = dict(case)
    seed, n, h, w, ch = (c.pop(k) for k in ("seed", "n", "h", "w", "c"))
    check(K.eltwise_case(seed, n, h, w, ch, **c), executor)


def test_conv_long_reduction_and_weight_zero_point_variants(executor):
    # sub-boxes (workloads) on the chunked kernel and on the kernels with pixel sums
    for kw in (dict(ic=256, k=(5, 5), pads=(2, 2, 2, 2)), dict(ic=128, k=(3, 3), pads=(1, 1, 1, 1), w_signed=False, w_zp=121),
               dict(ic=64, k=(1, 1), pads=(0, 0, 0, 0), w_signed=True, w_zp=-4)):
        ic = kw.pop("ic")
        full = K.conv_case(910 + ic, 2, 12, 10, ic, 64, **kw)
        want = K.run_oracle(full)
        tiled = K.conv_case(910 + ic, 2, 12, 10, ic, 64, variants=[((0, 0, 0), (9, 5, 31)), ((0, 6, 0), (9, 11, 31)),
                                                                    ((0, 0, 32), (4, 11, 63)), ((5, 0, 32), (9, 11, 63))], **kw)
        assert np.array_equal(K.run_hip(tiled, executor), want)


def _table_with(case, mults, shifts, biases):
    """Overwrite words [2] and [3] of the case's weight table, cycling through the given values per channel."""
    t = case.table.astype(np.int64)
    for c in range(t.shape[0]):
        t[c, 2] = (int(mults[c % len(mults)]) << 16) | (int(shifts[c % len(shifts)]) << 8)
        t[c, 3] = int(biases[c % len(biases)])
    case.table = (t & 0xFFFFFFFF).astype(np.uint32).view(np.int32).reshape(-1, 4).copy()
    return case


HI_SLOPES = [dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255),
             dict(mode=nce.PPE_LRELU, clamp_low=0, clamp_high=255),                                    # slope 0
             dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1023, lrelu_shift=11),  # just below 1/2
             dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1, lrelu_shift=1),      # 1/2: FP64 path
             dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=3, lrelu_shift=2),      # 3/4: FP64 path
             dict(mode=nce.PPE_LPRELU, clamp_low=3, clamp_high=250, lrelu_mult=1, lrelu_shift=31)]


@pytest.mark.parametrize("ppe", HI_SLOPES, ids=lambda p: f"m{p.get('lrelu_mult', '-')}s{p.get('lrelu_shift', '-')}")
@pytest.mark.parametrize("shift", [1, 15, 16, 17, 24, 31, 32, 33, 40, 44, 45, 46, 52, 53])
def test_conv_epilogue_shift_boundaries(executor, ppe, shift):
    # Every channel of a slice with the same shift: the integer high-word epilogue serves 16/17..32 (the multiplier
    # must fit 31 bits after scaling), FP64 or the 64-bit integer path the rest. Multipliers and biases at their
    # extremes; small shifts saturate.
    for out_signed, out_zp in ((False, 128), (True, -7), (False, 0)):
        lo, hi = (-128, 127) if out_signed else (0, 255)
        p = dict(ppe, clamp_low=max(lo, ppe["clamp_low"] + lo), clamp_high=min(hi, ppe["clamp_high"] + lo))
        case = K.conv_case(4000 + shift, 1, 9, 9, 64, 64, k=(1, 1), pads=(0, 0, 0, 0), ppe=p, out_signed=out_signed,
                           out_zp=out_zp)
        scale = 2.0 ** (shift - 22)   # keeps a part of the outputs inside the clamp range for every shift
        biases = [0, 1, -1, int(1000 * scale), -int(900 * scale), 2**31 - 1, -2**31, int(2**20 * scale), -int(2**20 * scale)]
        biases = [max(-2**31, min(2**31 - 1, b)) for b in biases]
        check(_table_with(case, [1, 16384, 32767, 65535, 0, 40000, 12345], [shift], biases), executor)


def test_conv_epilogue_mixed_shifts_in_one_slice(executor):
    # One channel outside the high-word range sends its whole slice to the FP64 epilogue; the other slice stays.
    case = K.conv_case(4100, 2, 7, 7, 128, 128, k=(3, 3), pads=(1, 1, 1, 1),
                       ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14))
    t = case.table.astype(np.int64)
    t[70, 2] = (20000 << 16) | (35 << 8)
    t[71, 2] = (65535 << 16) | (16 << 8)
    t[72, 3] = 2**31 - 1
    case.table = (t & 0xFFFFFFFF).astype(np.uint32).view(np.int32).reshape(-1, 4).copy()
    check(case, executor)


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("shift,mult", [(17, 65535), (17, 40000), (16, 32767), (16, 40000), (24, 1), (32, 65535), (33, 65535),
                                        (31, 16384), (26, 0)])
def test_eltwise_integer_path_boundaries(executor, signed, shift, mult):
    # the high-word form serves shifts up to 32 whose scaled multiplier fits 31 bits; input multipliers at both ends
    for in1, in2 in ((65535, 65535), (1, 65535), (0, 1), (20971, 31457)):
        # pick the input multipliers' common scale so that sums stay inside the output range for a part of the inputs
        zp = -5 if signed else 128
        check(K.eltwise_case(5000 + shift, 2, 5, 7, 48, signed=signed, zp_a=zp, zp_b=zp + 3, out_zp=zp, in1_mult=in1, in2_mult=in2,
                             mult=mult, shift=shift), executor)


def _conv_then_add(tuned, conv_kw, add_kw, conv_first, in_place, config="4,2,8,0", fuse=True, **more_env):
    """A convolution directly followed by the add that reads its output, through one task list; returns the two
    outputs from the GPU and from the oracle."""
    import torch
    env = dict(more_env)
    if config:
        env["NCE_HIP_CONV_WRES"] = config
    if not fuse:
        env["NCE_HIP_NO_FUSE"] = "1"
    executor = tuned(**env)
    c1 = K.conv_case(**conv_kw)
    y1 = K.run_oracle(c1)
    n, h, w, c = c1.out_shape
    c2 = K.eltwise_case(7001, n, h, w, c, signed=c1.out_signed, **add_kw)
    if conv_first:
        c2.input = y1
    else:
        c2.weights = y1
    y2 = K.run_oracle(c2)
    d1 = K.DeviceCase(c1)
    d2 = K.DeviceCase(c2)
    other = d2.weights if conv_first else d2.input
    out2 = other if in_place else d2.output
    t2 = K.build_task(c2, d1.output if conv_first else other, other if conv_first else d1.output, None, out2)
    tl = executor.task_list()
    tl.append(d1.task)
    tl.append(t2)
    stream = torch.cuda.current_stream().cuda_stream
    tl.enqueue(stream)
    executor.synchronize(stream)
    tl.destroy()
    return d1.output.cpu().numpy(), out2.cpu().numpy(), y1, y2


@pytest.mark.parametrize("conv_first,in_place", [(True, False), (False, False), (True, True), (False, True)])
@pytest.mark.parametrize("config", ["4,4,8,0", "4,2,8,0", "4,1,8,0", "2,2,8,0", None])
def test_conv_with_fused_residual_add(tuned, conv_first, in_place, config):
    # 1x1 convolutions that close a residual block, followed by the block's add: one launch for both on the 64-channel
    # kernels (a 32-channel configuration and the automatic choice fall back to two launches where they must).
    for ic, oc, out_signed, out_zp in ((64, 256, False, 128), (128, 80, True, -3), (256, 64, False, 0), (512, 128, False, 7)):
        lo, hi = (-128, 127) if out_signed else (0, 255)
        conv_kw = dict(seed=7100 + ic, n=2, h=9, w=11, ic=ic, oc=oc, k=(1, 1), pads=(0, 0, 0, 0), out_signed=out_signed, out_zp=out_zp,
                       ppe=dict(mode=nce.PPE_NOOP, clamp_low=lo + 5, clamp_high=hi))
        add_kw = dict(zp_a=out_zp, zp_b=(out_zp + 9) if not out_signed else -20, out_zp=out_zp, in1_mult=20971, in2_mult=31457,
                      mult=25600, shift=30)
        g1, g2, y1, y2 = _conv_then_add(tuned, conv_kw, add_kw, conv_first, in_place, config)
        assert np.array_equal(g1, y1), "convolution output"
        assert np.array_equal(g2, y2), "add output"


def test_conv_fused_add_equals_two_launches(tuned):
    # the same pair with the fusion switched off, and pairs the fusion must refuse (a 3x3 with padding, an add with a slope)
    conv_kw = dict(seed=7200, n=1, h=14, w=14, ic=128, oc=192, k=(1, 1), pads=(0, 0, 0, 0))
    add_kw = dict(zp_a=128, zp_b=100, out_zp=120)
    a = _conv_then_add(tuned, conv_kw, add_kw, True, False, "4,2,8,0", fuse=True)
    b = _conv_then_add(tuned, conv_kw, add_kw, True, False, "4,2,8,0", fuse=False)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    for conv_kw2, add_kw2 in ((dict(conv_kw, k=(3, 3), pads=(1, 1, 1, 1)), add_kw),
                              (conv_kw, dict(add_kw, ppe_extra=dict(mode=nce.PPE_LPRELU, lrelu_mult=1638, lrelu_shift=14))),
                              (conv_kw, dict(add_kw, shift=40))):
        g1, g2, y1, y2 = _conv_then_add(tuned, conv_kw2, add_kw2, False, False, "4,2,8,0")
        assert np.array_equal(g1, y1) and np.array_equal(g2, y2)


# ---- the limits the reference's verifier allows (kernel 1..11, stride 1..8, pad <= K/2, channels in 16s; VPUIP
# nce_invariant.cpp:1056-1108) and degenerate images --------------------------------------------------------------------

LIMIT_CONVS = [
    dict(n=1, h=11, w=11, ic=16, oc=16, k=(11, 11), s=(1, 1), pads=(5, 5, 5, 5)),      # largest kernel, largest padding
    dict(n=2, h=33, w=41, ic=32, oc=32, k=(11, 11), s=(8, 8), pads=(5, 5, 5, 5)),      # largest kernel and stride
    dict(n=1, h=24, w=17, ic=64, oc=48, k=(3, 3), s=(8, 1), pads=(1, 1, 1, 1)),        # strides 8 x 1
    dict(n=1, h=17, w=24, ic=64, oc=48, k=(3, 3), s=(1, 8), pads=(1, 1, 1, 1)),        # strides 1 x 8
    dict(n=1, h=1, w=1, ic=16, oc=16, k=(1, 1), s=(1, 1), pads=(0, 0, 0, 0)),          # one pixel, 16 channels
    dict(n=3, h=1, w=1, ic=2048, oc=1008, k=(1, 1), s=(1, 1), pads=(0, 0, 0, 0)),      # the classifier head: 1 x 1 images
    dict(n=1, h=3, w=3, ic=64, oc=64, k=(3, 3), s=(1, 1), pads=(0, 0, 0, 0)),          # one output pixel from a 3 x 3 image
    dict(n=2, h=1, w=37, ic=64, oc=32, k=(1, 3), s=(1, 1), pads=(1, 1, 0, 0)),         # one image row
    dict(n=2, h=37, w=1, ic=64, oc=32, k=(3, 1), s=(1, 1), pads=(0, 0, 1, 1)),         # one image column
    dict(n=1, h=2, w=2, ic=8192, oc=32, k=(1, 1), s=(1, 1), pads=(0, 0, 0, 0)),        # 8192 input channels
    dict(n=1, h=2, w=2, ic=64, oc=8192, k=(1, 1), s=(1, 1), pads=(0, 0, 0, 0)),        # 8192 output channels
    dict(n=1, h=1024, w=1024, ic=16, oc=16, k=(3, 3), s=(1, 1), pads=(1, 1, 1, 1)),    # a megapixel image
    dict(n=1, h=5, w=5, ic=16, oc=16, k=(5, 5), s=(1, 1), pads=(2, 0, 0, 2)),          # padding on two sides only
]


@pytest.mark.parametrize("c", LIMIT_CONVS, ids=lambda c: f"{c['n']}x{c['h']}x{c['w']}x{c['ic']}_{c['oc']}_k{c['k'][0]}x{c['k'][1]}s{c['s'][0]}x{c['s'][1]}")
def test_conv_limits(executor, c):
    check(K.conv_case(900 + c["ic"] % 97 + c["h"], c["n"], c["h"], c["w"], c["ic"], c["oc"], k=c["k"], s=c["s"], pads=c["pads"]), executor)


@pytest.mark.parametrize("kind", ["dw", "max", "avg"])
@pytest.mark.parametrize("h,w,c,k,s,pads", [(11, 11, 16, (11, 11), (1, 1), (5, 5, 5, 5)), (40, 33, 32, (11, 11), (8, 8), (5, 5, 5, 5)),
                                            (1, 1, 4096, (1, 1), (1, 1), (0, 0, 0, 0)), (1, 29, 48, (1, 3), (1, 2), (1, 1, 0, 0)),
                                            (29, 1, 48, (3, 1), (2, 1), (0, 0, 1, 1)), (700, 700, 16, (3, 3), (2, 2), (1, 1, 1, 1))])
def test_window_limits(executor, kind, h, w, c, k, s, pads):
    if kind == "dw":
        check(K.dw_case(950 + h, 1, h, w, c, k=k, s=s, pads=pads), executor)
    else:
        m, sh = K.approx(15, 1.0 / (k[0] * k[1]))
        ppe = None if kind == "max" else dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255, quant_mult=m, quant_shift=sh)
        check(K.pool_case(960 + h, kind == "max", 1, h, w, c, k=k, s=s, pads=pads, ppe=ppe), executor)


@pytest.mark.parametrize("n,h,w,c", [(1, 1, 1, 16), (1, 1, 1, 8192), (1, 1024, 1024, 16), (5, 3, 7, 48)])
def test_eltwise_limits(executor, n, h, w, c):
    check(K.eltwise_case(970 + c % 89, n, h, w, c), executor)
