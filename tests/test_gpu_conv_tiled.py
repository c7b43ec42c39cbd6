"""Parity of the LDS-tiled convolution kernel (many output channels) with the CPU oracle: every tile shape, forced
through NCE_HIP_CONV_TILED, on shapes that exercise tap masks, ragged channel and pixel tiles, weight sums, long
reductions, sub-boxes, permuted outputs and the fused residual add."""
import numpy as np
import pytest

import npu_plugin_amd as nce
from tests import cases as K
from tests.test_gpu_parity import check, _conv_then_add, _permuted_run

pytestmark = pytest.mark.gpu

TILED_SHAPES = [
    # (n, h, w, ic, oc, k, s, pads, in_zp)
    (2, 20, 20, 64, 64, (1, 1), (1, 1), (0, 0, 0, 0), 128),      # one reduction step
    (2, 20, 20, 256, 80, (1, 1), (1, 1), (0, 0, 0, 0), 5),       # weight sums, ragged channels
    (3, 19, 17, 64, 48, (3, 3), (1, 1), (1, 1, 1, 1), 128),      # tap masks, partial pixel tile
    (2, 21, 21, 128, 64, (3, 3), (2, 2), (1, 1, 1, 1), 200),     # stride 2 with masks and weight sums
    (1, 9, 9, 64, 16, (3, 3), (1, 1), (0, 0, 0, 0), 128),        # 3x3 without padding: every tap inside
    (2, 10, 10, 192, 144, (1, 1), (2, 2), (0, 0, 0, 0), 0),      # 1x1 stride 2, two channel tiles
    (2, 9, 9, 192, 272, (3, 3), (1, 1), (1, 1, 1, 1), 99),       # three channel tiles, the last one ragged
    (1, 5, 7, 2048, 48, (1, 1), (1, 1), (0, 0, 0, 0), 17),       # 32 steps, one partial pixel tile
    (1, 13, 11, 64, 160, (7, 7), (1, 1), (3, 3, 3, 3), 100),     # 49 taps: row / column validity bits
    (4, 30, 30, 64, 128, (3, 3), (1, 1), (1, 1, 1, 1), 128),     # many pixel tiles, images crossing tiles
    (2, 8, 8, 512, 512, (3, 3), (2, 2), (1, 1, 1, 1), 128),      # 72 steps, 4 x 4 output
    (2, 12, 12, 384, 96, (3, 3), (1, 1), (1, 1, 1, 1), 77),      # three 128-byte slices per tap, weight sums
    (2, 20, 20, 128, 64, (1, 1), (1, 1), (0, 0, 0, 0), 128),     # one 128-byte step
]


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("shape", TILED_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}s{s[6][0]}")
def test_conv_tiled_shapes(tuned, shape, tile):
    n, h, w, ic, oc, k, s, pads, in_zp = shape
    executor = tuned(NCE_HIP_CONV_TILED=tile)
    check(K.conv_case(1400 + ic + oc + h, n, h, w, ic, oc, k=k, s=s, pads=pads, in_zp=in_zp, out_zp=9,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=250, lrelu_mult=1638, lrelu_shift=14)), executor)


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5, 6])
def test_conv_tiled_types_and_modes(tuned, tile):
    executor = tuned(NCE_HIP_CONV_TILED=tile)
    wide = dict(k=(3, 3), pads=(1, 1, 1, 1))
    check(K.conv_case(1426, 2, 11, 11, 128, 160, in_signed=True, in_zp=-7, out_signed=True, out_zp=-128, **wide), executor)
    check(K.conv_case(1427, 2, 11, 11, 128, 64, w_signed=False, w_zp=128, in_zp=121, **wide), executor)
    check(K.conv_case(1428, 2, 11, 11, 128, 64, in_zp=3, ppe=dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255,
                                                                  round_mode=nce.ROUND_HALF_EVEN), **wide), executor)  # integer PPE path
    check(K.conv_case(1429, 2, 11, 11, 128, 64, in_zp=3, scale_lo=20.0, scale_hi=255.0, **wide), executor)           # may saturate int32
    check(K.conv_case(1430, 2, 11, 11, 128, 64, in_zp=250, ppe=dict(mode=nce.PPE_NOOP, clamp_low=128, clamp_high=255), **wide), executor)
    check(K.conv_case(1431, 2, 11, 11, 64, 64, in_zp=77, scale_lo=2e-13, scale_hi=9e-13, **wide), executor)          # shifts above 52
    check(K.conv_case(1432, 2, 11, 11, 64, 64, in_zp=77, scale_lo=1e-6, scale_hi=1e-5, **wide), executor)            # FP64 epilogue
    check(K.conv_case(1433, 2, 11, 11, 64, 64, in_zp=77, **wide,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=3, lrelu_shift=2)), executor)  # FP64 slope
    # weights whose zero point is not their storage offset: this kernel declines, the others take the task
    check(K.conv_case(1434, 2, 11, 11, 128, 64, in_zp=131, w_signed=False, w_zp=117, **wide), executor)
    # input channels that are no multiple of 64: declined as well
    check(K.conv_case(1435, 2, 11, 11, 48, 64, in_zp=131, **wide), executor)


@pytest.mark.parametrize("tile", [1, 2, 4, 5, 6])
def test_conv_tiled_variants_and_output_orders(tuned, tile):
    executor = tuned(NCE_HIP_CONV_TILED=tile)
    full = K.conv_case(1305, 2, 24, 20, 128, 192)
    want = K.run_oracle(full)
    tiled = K.conv_case(1305, 2, 24, 20, 128, 192, variants=[((0, 0, 0), (19, 11, 63)), ((0, 12, 0), (19, 23, 63)),
                                                             ((0, 0, 64), (9, 23, 191)), ((10, 0, 64), (19, 23, 191))])
    assert np.array_equal(K.run_hip(tiled, executor), want)
    part = K.conv_case(1305, 2, 24, 20, 128, 192, variants=[((3, 5, 64), (17, 20, 175))])
    canvas = np.full(part.out_shape, 0x5A, dtype=np.uint8)
    from oracle import nce_oracle
    nce_oracle.run(K.build_task(part, part.input, part.weights, part.table, canvas))
    assert np.array_equal(K.run_hip(part, executor), canvas)
    for order in ("nchw", "nwch"):
        got, want = _permuted_run(K.conv_case(1306, 2, 10, 10, 64, 144), order, executor)
        assert np.array_equal(got, want), order


@pytest.mark.parametrize("conv_first,in_place", [(True, False), (False, True)])
@pytest.mark.parametrize("tile", [1, 2, 3, 5, 6])
def test_conv_tiled_with_fused_residual_add(tuned, conv_first, in_place, tile):
    for ic, oc, out_signed, out_zp in ((64, 256, False, 128), (128, 80, True, -3), (512, 144, False, 7)):
        lo, hi = (-128, 127) if out_signed else (0, 255)
        conv_kw = dict(seed=7300 + ic, n=2, h=9, w=11, ic=ic, oc=oc, k=(1, 1), pads=(0, 0, 0, 0), out_signed=out_signed, out_zp=out_zp,
                       ppe=dict(mode=nce.PPE_NOOP, clamp_low=lo + 5, clamp_high=hi))
        add_kw = dict(zp_a=out_zp, zp_b=(out_zp + 9) if not out_signed else -20, out_zp=out_zp, in1_mult=20971, in2_mult=31457,
                      mult=25600, shift=30)
        g1, g2, y1, y2 = _conv_then_add(tuned, conv_kw, add_kw, conv_first, in_place, None, NCE_HIP_CONV_TILED=tile)
        assert np.array_equal(g1, y1), "convolution output"
        assert np.array_equal(g2, y2), "add output"
