"""Pins the oracle's per-element integer pipeline. The reference holds no executable implementation
and no golden output for it (it runs in NPU hardware), so it is pinned by what the mathematics fixes:
exact rational rounding, closed forms, an independent im2col/int64 formulation, torch's int64
conv2d / pooling, and identities between the task types. A dropped term, a wrong sign or index or a
transposed operand fails at least one of these."""
import ctypes as C
from fractions import Fraction

import numpy as np
import pytest

import npu_plugin_amd as nce
from npu_plugin_amd import _abi as abi
from oracle import nce_oracle as O
from tests import cases as K


# ---- (v) rounding: exact rational arithmetic ----------------------------------------------------

def exact_round(p, s, mode):
    q = Fraction(p, 2 ** s)
    if mode == abi.ROUND_NONE:
        return q.numerator // q.denominator
    if mode == abi.ROUND_HALF_EVEN:
        return round(q)  # Python rounds Fractions half to even
    return (q + Fraction(1, 2)).numerator // (q + Fraction(1, 2)).denominator  # floor(q + 1/2)


@pytest.mark.parametrize("mode", [abi.ROUND_HALF_UP, abi.ROUND_HALF_EVEN, abi.ROUND_NONE])
def test_rshift_round_boundaries_all_shifts(mode):
    for s in range(0, 64):
        half = 1 << (s - 1) if s else 0
        one = 1 << s
        pts = set()
        for k in (-3, -2, -1, 0, 1, 2, 3, 1000, -1000):
            for d in (-1, 0, 1):
                pts.add(k * one + half + d)
                pts.add(k * one + d)
        for p in pts:
            if abs(p) >= 2 ** 62:
                continue
            assert O.rshift_round(p, s, mode) == exact_round(p, s, mode), (p, s, mode)


def test_rshift_round_random():
    rng = np.random.default_rng(1)
    for _ in range(3000):
        s = int(rng.integers(0, 48))
        p = int(rng.integers(-2 ** 47, 2 ** 47))
        for mode in (0, 1, 2):
            assert O.rshift_round(p, s, mode) == exact_round(p, s, mode)


# ---- independent restatement of the PPE in Python integers --------------------------------------

def ppe_py(acc, bias, mult, shift, out_zp, out_signed, mode=abi.PPE_NOOP, clamp_low=abi.INT32_MIN,
           clamp_high=abi.INT32_MAX, lrelu_mult=1, lrelu_shift=0, round_mode=0, clamp_domain=0, **_):
    sat = lambda v: max(-2 ** 31, min(2 ** 31 - 1, v))
    x = sat(exact_round((acc + bias) * mult, shift, round_mode))
    pm, ps = {abi.PPE_LPRELU: (lrelu_mult, lrelu_shift), abi.PPE_LRELU: (0, 0), abi.PPE_LRELUX: (0, 0)}.get(mode, (1, 0))
    if x < 0:
        x = sat(exact_round(x * pm, ps, round_mode))
    if clamp_domain == abi.CLAMP_PRE_ZP:
        x = max(clamp_low, min(clamp_high, x)) + out_zp
    else:
        x = max(clamp_low, min(clamp_high, x + out_zp))
    lo, hi = (-128, 127) if out_signed else (0, 255)
    return max(lo, min(hi, x))


def _ppe_struct(**kw):
    t = nce.NCEClusterTask(abi.TASK_CONV, None)
    return t.addPPETask(**kw)


def test_ppe_scalar_against_python_integers():
    rng = np.random.default_rng(2)
    variants = [dict(), dict(mode=abi.PPE_LRELU), dict(mode=abi.PPE_LPRELU, lrelu_mult=1638, lrelu_shift=14),
                dict(mode=abi.PPE_LPRELU, lrelu_mult=-7, lrelu_shift=3, round_mode=1),
                dict(mode=abi.PPE_LRELUX, clamp_low=0, clamp_high=77), dict(clamp_low=-5, clamp_high=9, clamp_domain=1),
                dict(round_mode=2), dict(clamp_low=128, clamp_high=255)]
    for kw in variants:
        p = _ppe_struct(**kw)
        for _ in range(400):
            shift = int(rng.integers(0, 40))
            mult = int(rng.integers(0, 65536))
            acc = int(rng.integers(-2 ** 31, 2 ** 31)) if rng.random() < 0.3 else int(rng.integers(-300000, 300000))
            bias = int(rng.integers(-5000, 5000))
            zp = int(rng.integers(0, 256))
            got = O.ppe(acc, bias, mult, shift, p, zp, abi.DT_U8)
            assert got == ppe_py(acc, bias, mult, shift, zp, False, **kw), (kw, acc, bias, mult, shift, zp)
            zps = zp - 128
            assert O.ppe(acc, bias, mult, shift, p, zps, abi.DT_I8) == ppe_py(acc, bias, mult, shift, zps, True, **kw)


def test_ppe_int32_saturation_between_stages():
    # shift 0 and a huge accumulator: the requantized value saturates to int32 BEFORE the PReLU slope
    p = _ppe_struct(mode=abi.PPE_LPRELU, lrelu_mult=1, lrelu_shift=31)
    assert O.ppe(-2 ** 31, 0, 65535, 0, p, 128, abi.DT_U8) == 127  # sat(-2^31) * 1 >> 31 = -1 ; -1 + 128
    assert ppe_py(-2 ** 31, 0, 65535, 0, 128, False, mode=abi.PPE_LPRELU, lrelu_mult=1, lrelu_shift=31) == 127


# ---- (i) closed form --------------------------------------------------------------------------

def test_closed_form_1x1_unit_weights_exhaustive_over_byte_values():
    # 1x1 conv, all weights 1, scale 16384 >> 14 = 1: out = clamp(sum_ic (a - zp) + bias + zp_out)
    ic, oc, zp_in, zp_out = 16, 16, 100, 7
    x = np.zeros((1, 16, 16, ic), dtype=np.uint8)
    x[0].reshape(256, ic)[:, :] = np.arange(256, dtype=np.uint8)[:, None]          # every byte value once
    x[0].reshape(256, ic)[:, 1:] = (np.arange(256)[:, None] * np.arange(1, ic)[None, :] % 251).astype(np.uint8)
    w = np.ones((oc, 1, 1, ic), dtype=np.int8)
    table = np.zeros((oc, 4), dtype=np.int32)
    table[:, 2] = (16384 << 16) | (14 << 8)
    table[:, 3] = np.arange(oc) * 37 - 300
    case = K.Case("closed", abi.TASK_CONV, x, (1, 16, 16, oc), zp_in, zp_out, False, w, 0, table, (1, 1), (1, 1),
                  (0, 0, 0, 0), dict(clamp_low=0, clamp_high=255))
    got = K.run_oracle(case)
    s = (x.astype(np.int64) - zp_in).sum(axis=3, keepdims=True) + table[:, 3][None, None, None, :] + zp_out
    assert np.array_equal(got, np.clip(s, 0, 255).astype(np.uint8))


# ---- (ii) independent im2col / int64 GEMM formulation -----------------------------------------

def conv_im2col(case):
    x = case.input.astype(np.int64) - case.in_zp
    n, h, w, ic = x.shape
    ky, kx = case.kernel
    sy, sx = case.strides
    pl, pr, pt, pb = case.pads
    xp = np.zeros((n, h + pt + pb, w + pl + pr, ic), dtype=np.int64)      # zero AFTER zero-point removal
    xp[:, pt:pt + h, pl:pl + w] = x
    _, oh, ow, oc = case.out_shape
    cols = np.empty((n, oh, ow, ky, kx, ic), dtype=np.int64)
    for a in range(ky):
        for b in range(kx):
            cols[:, :, :, a, b] = xp[:, a:a + (oh - 1) * sy + 1:sy, b:b + (ow - 1) * sx + 1:sx]
    wm = (case.weights.astype(np.int64) - case.w_zp).reshape(oc, -1)
    return cols.reshape(n * oh * ow, -1) @ wm.T                            # [pixels, oc]


def requant_table(acc, case):
    n, oh, ow, oc = case.out_shape
    out = np.empty((n * oh * ow, oc), dtype=np.int64)
    for c in range(oc):
        w2 = int(case.table[c, 2]) & 0xFFFFFFFF
        mult, shift, bias = w2 >> 16, (w2 >> 8) & 0x3F, int(case.table[c, 3])
        out[:, c] = [ppe_py(int(a), bias, mult, shift, case.out_zp, case.out_signed, **case.ppe) for a in acc[:, c]]
    return out.reshape(n, oh, ow, oc).astype(np.int8 if case.out_signed else np.uint8)


CONV_SHAPES = [dict(k=(3, 3), s=(1, 1), pads=(1, 1, 1, 1)), dict(k=(1, 1), s=(2, 2), pads=(0, 0, 0, 0)),
               dict(k=(5, 3), s=(2, 1), pads=(1, 0, 2, 1)), dict(k=(7, 7), s=(2, 2), pads=(3, 3, 3, 3)),
               dict(k=(2, 2), s=(1, 1), pads=(1, 1, 1, 1))]


@pytest.mark.parametrize("shape", CONV_SHAPES, ids=lambda s: f"k{s['k'][0]}x{s['k'][1]}s{s['s'][0]}")
@pytest.mark.parametrize("types", [dict(), dict(in_signed=True, in_zp=-9, out_signed=True, out_zp=3),
                                   dict(w_signed=False, w_zp=119, in_zp=7)])
def test_conv_against_im2col(shape, types):
    case = K.conv_case(5, 2, 9, 8, 16, 16, ppe=dict(mode=abi.PPE_LPRELU, clamp_low=-128 if types.get("out_signed") else 0,
                                                    clamp_high=127 if types.get("out_signed") else 255, lrelu_mult=1638,
                                                    lrelu_shift=14), **shape, **types)
    assert np.array_equal(K.run_oracle(case), requant_table(conv_im2col(case), case))


# ---- (iii) torch int64 library routines ----------------------------------------------------------

def test_conv_accumulators_against_torch_conv2d():
    import torch
    case = K.conv_case(6, 2, 12, 10, 32, 16, k=(3, 3), s=(2, 2), pads=(1, 1, 1, 1), in_zp=0, out_zp=0)
    # symmetric padding and zero input zero point: F.conv2d on int64 is the same sum
    x = torch.from_numpy(case.input.astype(np.int64)).permute(0, 3, 1, 2)
    w = torch.from_numpy(case.weights.astype(np.int64)).permute(0, 3, 1, 2)
    acc = torch.nn.functional.conv2d(x, w, stride=2, padding=1).permute(0, 2, 3, 1).reshape(-1, 16).numpy()
    assert np.array_equal(acc, conv_im2col(case))
    assert np.array_equal(K.run_oracle(case), requant_table(acc, case))


def test_maxpool_against_torch():
    import torch
    case = K.pool_case(7, True, 2, 13, 11, 32)
    x = torch.from_numpy(case.input.astype(np.int64)).permute(0, 3, 1, 2).double()
    ref = torch.nn.functional.max_pool2d(x, 3, 2, 1).permute(0, 2, 3, 1).numpy().astype(np.uint8)
    assert np.array_equal(K.run_oracle(case), ref)


def test_avgpool_against_torch_sum_pool():
    import torch
    case = K.pool_case(8, False, 2, 12, 12, 16, k=(3, 3), s=(1, 1), pads=(1, 1, 1, 1), in_zp=17, out_zp=5)
    x = torch.from_numpy(case.input.astype(np.float64) - 17).permute(0, 3, 1, 2)
    sums = (torch.nn.functional.avg_pool2d(x, 3, 1, 1, count_include_pad=True) * 9).round().permute(0, 2, 3, 1).numpy()
    m, s = case.ppe["quant_mult"], case.ppe["quant_shift"]
    ref = np.vectorize(lambda a: ppe_py(int(a), 0, m, s, 5, False, clamp_low=0, clamp_high=255))(sums)
    assert np.array_equal(K.run_oracle(case), ref.astype(np.uint8))


def test_eltwise_against_numpy():
    case = K.cfg4(n=1)
    a = case.input.astype(np.int64) - 120
    b = case.weights.astype(np.int64) - 130
    acc = 20971 * a + 31457 * b
    y = ((acc * 25600 + (1 << 29)) >> 30) + 128
    assert np.array_equal(K.run_oracle(case), np.clip(y, 0, 255).astype(np.uint8))
    # real-valued meaning: 0.02*(a) + 0.03*(b) = 0.04*(q-128) within one quantization step
    real = (0.02 * a + 0.03 * b) / 0.04 + 128
    assert np.abs(np.clip(real, 0, 255) - K.run_oracle(case)).max() <= 1.0


# ---- (iv) identities between task types ---------------------------------------------------------

def test_dwconv_equals_conv_with_block_diagonal_weights():
    dw = K.dw_case(9, 1, 10, 9, 16, k=(3, 3), s=(1, 1), in_zp=11, out_zp=200)
    full = np.zeros((16, 3, 3, 16), dtype=np.int8)
    for c in range(16):
        full[c, :, :, c] = dw.weights[c, :9].reshape(3, 3)
    conv = K.Case("bd", abi.TASK_CONV, dw.input, dw.out_shape, dw.in_zp, dw.out_zp, False, full, 0, dw.table, (3, 3),
                  (1, 1), dw.pads, dw.ppe)
    assert np.array_equal(K.run_oracle(dw), K.run_oracle(conv))


def test_avgpool_equals_dwconv_with_unit_weights():
    avg = K.pool_case(10, False, 1, 12, 12, 16, k=(2, 2), s=(2, 2), pads=(0, 0, 0, 0), in_zp=9, out_zp=1)
    w = np.zeros((16, 16), dtype=np.int8)
    w[:, :4] = 1
    table = np.zeros((16, 4), dtype=np.int32)
    table[:, 2] = (avg.ppe["quant_mult"] << 16) | (avg.ppe["quant_shift"] << 8)
    dw = K.Case("dw1", abi.TASK_DWCONV, avg.input, avg.out_shape, 9, 1, False, w, 0, table, (2, 2), (2, 2),
                (0, 0, 0, 0), dict(clamp_low=0, clamp_high=255))
    assert np.array_equal(K.run_oracle(avg), K.run_oracle(dw))


def test_eltwise_commutes_and_clamp_domains_agree():
    c = K.eltwise_case(11, 1, 6, 6, 32, in1_mult=20000, in2_mult=20000, zp_a=9, zp_b=9)
    swapped = K.eltwise_case(11, 1, 6, 6, 32, in1_mult=20000, in2_mult=20000, zp_a=9, zp_b=9)
    swapped.input, swapped.weights = c.weights, c.input
    assert np.array_equal(K.run_oracle(c), K.run_oracle(swapped))
    pre = K.eltwise_case(11, 1, 6, 6, 32, out_zp=100, ppe_extra=dict(clamp_low=-100, clamp_high=155, clamp_domain=1))
    post = K.eltwise_case(11, 1, 6, 6, 32, out_zp=100, ppe_extra=dict(clamp_low=0, clamp_high=255, clamp_domain=0))
    assert np.array_equal(K.run_oracle(pre), K.run_oracle(post))


def test_relu_forms_agree():
    """A quantized ReLU as mode LRELU and as NOOP with clamp_low = zp (the 37XX form) give the same bytes."""
    a = K.conv_case(12, 1, 8, 8, 16, 16, ppe=dict(mode=abi.PPE_LRELU, clamp_low=0, clamp_high=255))
    b = K.conv_case(12, 1, 8, 8, 16, 16, ppe=dict(mode=abi.PPE_NOOP, clamp_low=128, clamp_high=255))
    ya = K.run_oracle(a)
    assert np.array_equal(ya, K.run_oracle(b)) and (ya >= 128).all() and (ya > 128).any()


def test_variant_split_invariance_and_untouched_bytes():
    full = K.conv_case(13, 2, 8, 8, 16, 32)
    want = K.run_oracle(full)
    split = K.conv_case(13, 2, 8, 8, 16, 32, variants=[((0, 0, 0), (7, 3, 15)), ((0, 4, 0), (7, 7, 15)),
                                                       ((0, 0, 16), (4, 7, 31)), ((5, 0, 16), (7, 7, 31))])
    assert np.array_equal(K.run_oracle(split), want)
    part = K.conv_case(13, 2, 8, 8, 16, 32, variants=[((2, 1, 16), (5, 6, 31))])
    canvas = np.full(part.out_shape, 0xEE, dtype=np.uint8)
    O.run(K.build_task(part, part.input, part.weights, part.table, canvas))
    assert np.array_equal(canvas[:, 1:7, 2:6, 16:], want[:, 1:7, 2:6, 16:])
    canvas[:, 1:7, 2:6, 16:] = 0xEE
    assert (canvas == 0xEE).all()


def test_padding_contributes_nothing_even_with_nonzero_zero_point():
    # a constant image equal to the zero point gives acc = 0 everywhere, borders included
    x = np.full((1, 6, 6, 16), 77, dtype=np.uint8)
    rng = np.random.default_rng(3)
    w = rng.integers(-127, 128, size=(16, 3, 3, 16)).astype(np.int8)
    table = np.zeros((16, 4), dtype=np.int32)
    table[:, 2] = (16384 << 16) | (14 << 8)
    table[:, 3] = np.arange(16)
    case = K.Case("pad", abi.TASK_CONV, x, (1, 6, 6, 16), 77, 10, False, w, 0, table, (3, 3), (1, 1), (1, 1, 1, 1),
                  dict(clamp_low=0, clamp_high=255))
    assert np.array_equal(K.run_oracle(case), np.broadcast_to(np.arange(16, dtype=np.uint8) + 10, (1, 6, 6, 16)))


def test_outputs_are_not_degenerate():
    """The benchmark configurations exercise the requantizer: outputs spread over the byte range."""
    for case in (K.cfg1(), K.cfg2(n=1), K.cfg3_dw(n=1), K.cfg4(n=1)):
        y = K.run_oracle(case)
        assert len(np.unique(y)) > 200, case.name
