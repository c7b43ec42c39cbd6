"""Parity of the patch convolution kernel (weights slice and the patch's input pixels both in LDS) with the CPU oracle:
forced through NCE_HIP_CONV_PATCH, automatic and forced shapes (channel fragments per slice, output rows per patch), on
shapes that exercise the halo fill at every image border, ragged last fragments, last patches with fewer rows, one and
two patch buffers, several patches per workgroup, every pixel width (64 .. 1024 input channels), weight sums, u8 weights,
sub-boxes and permuted outputs. Shapes the kernel declines (stride 2, other channel counts, weights whose zero point is
not their storage offset) must still give the oracle's bytes through the kernels that take them instead."""
import numpy as np
import pytest

import npu_plugin_amd as nce
from tests import cases as K
from tests.test_gpu_parity import check, _permuted_run

pytestmark = pytest.mark.gpu

PATCH_SHAPES = [
    # (n, h, w, ic, oc, k, pads, in_zp)
    (2, 20, 20, 64, 64, (3, 3), (1, 1, 1, 1), 128),       # the plain case
    (3, 19, 17, 64, 48, (3, 3), (1, 1, 1, 1), 5),         # odd sizes, ragged channels, weight sums
    (1, 9, 9, 64, 16, (3, 3), (0, 0, 0, 0), 128),         # no padding: nothing outside the image
    (2, 14, 14, 256, 96, (3, 3), (1, 1, 1, 1), 200),      # a pixel as wide as the banks
    (2, 7, 7, 512, 64, (3, 3), (1, 1, 1, 1), 128),        # two bank windows per pixel
    (1, 6, 5, 1024, 32, (3, 3), (1, 1, 1, 1), 99),        # four windows, 144 steps
    (2, 28, 28, 128, 128, (3, 3), (1, 1, 1, 1), 128),     # two slices
    (1, 13, 11, 64, 80, (5, 5), (2, 2, 2, 2), 100),       # 25 taps
    (2, 12, 16, 128, 64, (2, 2), (0, 1, 0, 1), 128),      # even kernel, one-sided padding
    (1, 10, 33, 64, 64, (1, 3), (1, 1, 0, 0), 77),        # one kernel row
    (1, 33, 10, 64, 64, (3, 1), (0, 0, 1, 1), 77),        # one kernel column
    (4, 56, 56, 64, 64, (3, 3), (1, 1, 1, 1), 128),       # several patches per image
    (40, 12, 12, 64, 64, (3, 3), (1, 1, 1, 1), 128),      # more patches than workgroups: two buffers in flight
    (2, 20, 20, 64, 64, (1, 1), (0, 0, 0, 0), 128),       # 1x1: no halo at all
]


def _id(s):
    return f"{s[0]}x{s[1]}x{s[2]}x{s[3]}_{s[4]}_k{s[5][0]}x{s[5][1]}"


@pytest.mark.parametrize("knob", ["1", "4,1", "4,3", "2,5", "2,64", "4,3,16", "2,6,16", "2,14,16,1"])
@pytest.mark.parametrize("shape", PATCH_SHAPES, ids=_id)
def test_conv_patch_shapes(tuned, shape, knob):
    n, h, w, ic, oc, k, pads, in_zp = shape
    executor = tuned(NCE_HIP_CONV_PATCH=knob)
    check(K.conv_case(2400 + ic + oc + h, n, h, w, ic, oc, k=k, s=(1, 1), pads=pads, in_zp=in_zp, out_zp=9,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=250, lrelu_mult=1638, lrelu_shift=14)), executor)


@pytest.mark.parametrize("knob", ["1", "4,2", "2,3", "4,2,16"])
def test_conv_patch_types_and_modes(tuned, knob):
    executor = tuned(NCE_HIP_CONV_PATCH=knob)
    wide = dict(k=(3, 3), pads=(1, 1, 1, 1))
    check(K.conv_case(2426, 2, 11, 11, 128, 160, in_signed=True, in_zp=-7, out_signed=True, out_zp=-128, **wide), executor)
    check(K.conv_case(2427, 2, 11, 11, 128, 64, w_signed=False, w_zp=128, in_zp=121, **wide), executor)
    check(K.conv_case(2428, 2, 11, 11, 128, 64, in_zp=3, ppe=dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255,
                                                                  round_mode=nce.ROUND_HALF_EVEN), **wide), executor)  # integer PPE path
    check(K.conv_case(2429, 2, 11, 11, 128, 64, in_zp=3, scale_lo=20.0, scale_hi=255.0, **wide), executor)           # may saturate int32
    check(K.conv_case(2430, 2, 11, 11, 128, 64, in_zp=250, ppe=dict(mode=nce.PPE_NOOP, clamp_low=128, clamp_high=255), **wide), executor)
    check(K.conv_case(2431, 2, 11, 11, 64, 64, in_zp=77, scale_lo=2e-13, scale_hi=9e-13, **wide), executor)          # shifts above 52
    check(K.conv_case(2432, 2, 11, 11, 64, 64, in_zp=77, scale_lo=1e-6, scale_hi=1e-5, **wide), executor)            # FP64 epilogue
    check(K.conv_case(2433, 2, 11, 11, 64, 64, in_zp=77, **wide,
                      ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=3, lrelu_shift=2)), executor)  # FP64 slope
    # declined by this kernel, taken by the others: weights zero point away from the storage offset, input channels that
    # are no power of two from 64 up, stride 2
    check(K.conv_case(2434, 2, 11, 11, 128, 64, in_zp=131, w_signed=False, w_zp=117, **wide), executor)
    check(K.conv_case(2435, 2, 11, 11, 48, 64, in_zp=131, **wide), executor)
    check(K.conv_case(2436, 2, 11, 11, 192, 64, in_zp=131, **wide), executor)
    check(K.conv_case(2437, 2, 21, 21, 128, 64, s=(2, 2), in_zp=131, **wide), executor)


@pytest.mark.parametrize("knob", ["1", "4,5", "2,2"])
def test_conv_patch_variants_and_output_orders(tuned, knob):
    executor = tuned(NCE_HIP_CONV_PATCH=knob)
    full = K.conv_case(2305, 2, 24, 20, 128, 192)
    want = K.run_oracle(full)
    tiled = K.conv_case(2305, 2, 24, 20, 128, 192, variants=[((0, 0, 0), (19, 11, 63)), ((0, 12, 0), (19, 23, 63)),
                                                             ((0, 0, 64), (9, 23, 191)), ((10, 0, 64), (19, 23, 191))])
    assert np.array_equal(K.run_hip(tiled, executor), want)
    part = K.conv_case(2305, 2, 24, 20, 128, 192, variants=[((3, 5, 64), (17, 20, 175))])
    canvas = np.full(part.out_shape, 0x5A, dtype=np.uint8)
    from oracle import nce_oracle
    nce_oracle.run(K.build_task(part, part.input, part.weights, part.table, canvas))
    assert np.array_equal(K.run_hip(part, executor), canvas)
    for order in ("nchw", "nwch"):
        got, want = _permuted_run(K.conv_case(2306, 2, 10, 10, 64, 144), order, executor)
        assert np.array_equal(got, want), order


def test_conv_patch_is_what_ran(tuned):
    """The knob must select the kernel (a test that passes on another kernel proves nothing about this one)."""
    executor = tuned(log_level=3, NCE_HIP_CONV_PATCH="1")
    check(K.conv_case(2500, 2, 20, 20, 64, 64), executor)
    assert "patch kernel" in executor.log()
