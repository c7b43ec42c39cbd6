"""Parameter generation against the known-answer values held by the reference's lit tests
(tests/golden/param_kats.json). Both implementations are checked: the oracle's C restatement and
the product's nce_params.h library; neither is used to check the other."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from npu_plugin_amd import _abi as abi
from oracle import nce_oracle as O

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "param_kats.json")))
MODES = {"NOOP": abi.PPE_NOOP, "ADD": abi.PPE_ADD, "LRELU": abi.PPE_LRELU, "LRELUX": abi.PPE_LRELUX, "LPRELU": abi.PPE_LPRELU}


def lib_eltwise(s1, s2, so, arch=abi.ARCH_VPUX37XX):
    v = [C.c_int32() for _ in range(4)]
    rc = abi.load_library().nceEltwiseQuantApproximate(arch, s1, s2, so, *[C.byref(x) for x in v])
    assert rc == abi.SUCCESS
    return tuple(x.value for x in v)


def lib_quant(t, arch=abi.ARCH_VPUX37XX):
    v = [C.c_int32() for _ in range(3)]
    assert abi.load_library().nceQuantApproximate(arch, t, *[C.byref(x) for x in v]) == abi.SUCCESS
    return tuple(x.value for x in v)


def lib_prelu(a, arch):
    v = [C.c_int32() for _ in range(2)]
    assert abi.load_library().ncePReLUApproximate(arch, a, *[C.byref(x) for x in v]) == abi.SUCCESS
    return tuple(x.value for x in v)


@pytest.mark.parametrize("k", KATS["eltwise_approx_37xx"], ids=lambda k: k["source"].split("/")[-1])
def test_eltwise_approximation(k):
    want = (k["in1_mult"], k["in2_mult"], k["mult"], k["shift"])
    assert O.eltwise_approx(k["in1_scale"], k["in2_scale"], k["out_scale"]) == want
    assert lib_eltwise(k["in1_scale"], k["in2_scale"], k["out_scale"]) == want


@pytest.mark.parametrize("k", KATS["prelu_approx"], ids=lambda k: k["arch"])
def test_prelu_approximation(k):
    arch = 1 if k["arch"] == "37XX" else 0
    assert O.prelu_approx(k["alpha"], arch) == (k["mult"], k["shift"])
    assert lib_prelu(k["alpha"], arch) == (k["mult"], k["shift"])


def test_quant_approximation():
    for k in KATS["quant_approx"]:
        assert O.quant_approx(k["target"], 0)[:2] == (k["mult"], k["shift"])
        assert lib_quant(k["target"], 0)[:2] == (k["mult"], k["shift"])
    for k in KATS["survey_examples"]:
        if "target" in k:
            assert O.quant_approx(k["target"])[:2] == (k["mult"], k["shift"])
            assert lib_quant(k["target"])[:2] == (k["mult"], k["shift"])
        else:
            want = (k["in1_mult"], k["in2_mult"], k["mult"], k["shift"])
            assert O.eltwise_approx(*k["eltwise"]) == want and lib_eltwise(*k["eltwise"]) == want


def test_approximation_edge_cases():
    # mantissa is truncated, never rounded: 15 bits of 0.7 = floor(0.7 * 32768 * ...) after frexp
    m, s, p = O.approximate(15, 0.7)
    assert (m, s, p) == (22937, 15, 0) and 22937 == int(0.7 * 2 ** 15)
    assert O.approximate(15, 0.0) == (0, 15, 0)
    # exponent above the mantissa width -> post shift (refused on 37XX, allowed on 30XX)
    assert O.approximate(15, float(2 ** 17)) == (16384, 0, -3)
    with pytest.raises(ValueError):
        O.quant_approx(float(2 ** 17), 1)
    assert O.quant_approx(float(2 ** 17), 0) == (16384, 0, -3)
    v = [C.c_int32() for _ in range(3)]
    assert abi.load_library().nceQuantApproximate(1, float(2 ** 17), *[C.byref(x) for x in v]) == abi.ERROR_INVALID_ARGUMENT
    # mult stays in [16384, 32767] for every positive normal target
    for t in (1e-9, 3.3e-4, 0.5, 0.999999, 1.0, 1.5, 255.0, 32767.9):
        m, s, _ = O.approximate(15, t)
        assert 16384 <= m <= 32767
        assert abs(m / 2.0 ** s - t) / t < 2 ** -14


def test_eltwise_shift_down_branch_and_refusal():
    # shifts too far apart to scale the smaller multiplier up -> larger one is scaled down
    got = O.eltwise_approx(1e-6, 0.9, 1.0)
    assert got == lib_eltwise(1e-6, 0.9, 1.0)
    m1, m2, mo, so = got
    assert m1 == 0 and 16384 <= m2 <= 32767 and so == 14 + 15
    with pytest.raises(ValueError):
        O.eltwise_approx(1e-12, 1e-12, 1e9)


def test_weight_table_words():
    for k in KATS["table_word2_37xx_int"]:
        t = O.weights_table(k["oc"], 0, k["ptr_step"], k["in_scale"], k["out_scale"], [k["w_scale"]],
                            sparsity_ptr=k["sparsity_ptr"])
        for c in range(k["oc"]):
            assert t[c].tolist() == [c * k["ptr_step"], k["sparsity_ptr"], k["word2"], 0]
        import numpy as np
        out = np.zeros((k["oc"], 4), dtype=np.int32)
        ws = (C.c_double * 1)(k["w_scale"])
        rc = abi.load_library().nceWeightsTableFill(1, k["oc"], 0, k["ptr_step"], k["sparsity_ptr"], k["in_scale"],
                                                    k["out_scale"], ws, 1, None, out.ctypes.data_as(C.POINTER(C.c_int32)))
        assert rc == abi.SUCCESS and (out == t).all()
    assert O.lib().nce_oracle_scale_word(1, 14, 16384, -1) == 1073745408 == (14 << 8) + (16384 << 16)
    # 30XX adds prelu_scale = 1 at bit 0 and round_mode = 1 at bit 14; LPRELU overwrites the low byte
    assert O.lib().nce_oracle_scale_word(0, 14, 16384, -1) == 1073745408 | 1 | (1 << 14)
    assert O.lib().nce_oracle_scale_word(0, 14, 16384, 102) & 0xFF == 102


def test_float_bits():
    a, b = KATS["float_bits_37xx"]
    assert O.lib().nce_oracle_float_bits(a["value"]) == a["bits"]
    assert O.lib().nce_oracle_float_bits(1.0 / b["value_reciprocal_of"]) == b["bits"]


def test_bias_rescale_rounds_half_away_from_zero_and_refuses_overflow():
    out = C.c_int32()
    L = O.lib()
    assert L.nce_oracle_rescaled_bias(2.5, 1.0, 1.0, C.byref(out)) == 0 and out.value == 3
    assert L.nce_oracle_rescaled_bias(-2.5, 1.0, 1.0, C.byref(out)) == 0 and out.value == -3
    assert L.nce_oracle_rescaled_bias(1.0, 0.078737745098039214, 1.0, C.byref(out)) == 0 and out.value == 13
    assert L.nce_oracle_rescaled_bias(3e9, 1.0, 1.0, C.byref(out)) == -1
    import numpy as np
    t = np.zeros((2, 4), dtype=np.int32)
    ws = (C.c_double * 2)(0.5, 0.25)
    bias = (C.c_double * 2)(1.25, -1.25)
    assert abi.load_library().nceWeightsTableFill(1, 2, 0, 16, 0xFFFFFF, 0.5, 1.0, ws, 2, bias,
                                                  t.ctypes.data_as(C.POINTER(C.c_int32))) == abi.SUCCESS
    assert t[:, 3].tolist() == [5, -10] and t[:, 0].tolist() == [0, 16] and t[:, 1].tolist() == [0xFFFFFF] * 2
    assert (O.weights_table(2, 0, 16, 0.5, 1.0, [0.5, 0.25], bias=[1.25, -1.25]) == t).all()


@pytest.mark.parametrize("k", KATS["setup_ppe_37xx"], ids=lambda k: k["name"])
def test_setup_ppe_rewrite(k):
    p = abi.PpeTask()
    p.mode = abi.PPE_ADD
    p.clamp_low, p.clamp_high = k["in"]["low"], k["in"]["high"]
    p.lrelu_mult, p.lrelu_shift = k["in"]["lrelu_mult"], k["in"]["lrelu_shift"]
    O.lib().nce_oracle_ppe_stage2_37xx(1, 0, 255, k["out_zp"], C.byref(p))
    assert (p.mode, p.clamp_low, p.clamp_high) == (MODES[k["out"]["mode"]], k["out"]["low"], k["out"]["high"])
    assert p.clamp_domain == abi.CLAMP_POST_ZP


def test_ppe_from_postop_pipeline():
    """stage 1 + stage 2 end to end in the product library vs the oracle, and vs the lit values where
    they exist (ReLU on u8 zp 128 -> NOOP [128,255]; no post-op -> NOOP [0,255]; LeakyReLU 0.1 -> LPRELU 1638/14)."""
    lib = abi.load_library()
    for postop, p0, p1, zp, want in [
        (abi.POSTOP_RELU, 0, 0, 128, (abi.PPE_NOOP, 128, 255, 1, 0)),
        (abi.POSTOP_RELU, 0, 0, 0, (abi.PPE_NOOP, 0, 255, 1, 0)),
        (abi.POSTOP_NONE, 0, 0, 128, (abi.PPE_NOOP, 0, 255, 1, 0)),
        (abi.POSTOP_LEAKY_RELU, 0.1, 0, 128, (abi.PPE_LPRELU, 0, 255, 1638, 14)),
        (abi.POSTOP_LEAKY_RELU, 0.0, 0, 3, (abi.PPE_LPRELU, 0, 255, 0, 0)),
        (abi.POSTOP_CLAMP, 0.0, 6.0, 0, (abi.PPE_LRELUX, 0, 60, 1, 0)),
        (abi.POSTOP_CLAMP, -1.0, 1.0, 128, (abi.PPE_NOOP, 118, 138, 1, 0)),
    ]:
        q = abi.Quant(0.1, zp, abi.DT_U8)
        got = abi.PpeTask()
        assert lib.ncePpeFromPostOp(abi.ARCH_VPUX37XX, postop, p0, p1, q, C.byref(got)) == abi.SUCCESS
        assert (got.mode, got.clamp_low, got.clamp_high, got.lrelu_mult, got.lrelu_shift) == want, (postop, zp)
        ref = abi.PpeTask()
        assert O.lib().nce_oracle_ppe_stage1(1, postop, p0, p1, 0, 255, 0.1, zp, C.byref(ref)) == 0
        O.lib().nce_oracle_ppe_stage2_37xx(int(postop != abi.POSTOP_NONE), 0, 255, zp, C.byref(ref))
        assert (ref.mode, ref.clamp_low, ref.clamp_high, ref.lrelu_mult, ref.lrelu_shift) == want


def test_avgpool_and_eltwise_ppe_generators():
    lib = abi.load_library()
    for k in KATS["avgpool_scale"]:
        assert O.lib().nce_oracle_avgpool_scale(1.0, 1.0, k["ky"], k["kx"]) == pytest.approx(k["scale"], abs=0, rel=1e-15)
    p = abi.PpeTask()
    q = abi.Quant(0.5, 128, abi.DT_U8)
    assert lib.ncePpeForAvgPool(1, q, q, 2, 2, abi.POSTOP_NONE, 0, 0, C.byref(p)) == abi.SUCCESS
    assert (p.has_quant, p.quant_mult, p.quant_shift, p.mode, p.clamp_low, p.clamp_high) == (1, 16384, 16, abi.PPE_NOOP, 0, 255)
    k = KATS["eltwise_approx_37xx"][3]  # the setup_ppe lit case: ReLU, out zp 128
    p = abi.PpeTask()
    rc = lib.ncePpeForEltwiseAdd(1, abi.Quant(k["in1_scale"], 0, abi.DT_U8), abi.Quant(k["in2_scale"], 0, abi.DT_U8),
                                 abi.Quant(k["out_scale"], 128, abi.DT_U8), abi.POSTOP_RELU, 0, 0, C.byref(p))
    assert rc == abi.SUCCESS
    assert (p.mode, p.clamp_low, p.clamp_high, p.quant_mult, p.quant_shift, p.in1_quant_mult, p.in2_quant_mult) == \
        (abi.PPE_NOOP, 128, 255, k["mult"], k["shift"], k["in1_mult"], k["in2_mult"])
    # 30XX: one scale in1/out, mode stays ADD, clamps stay in the zero-point-free domain
    p = abi.PpeTask()
    assert lib.ncePpeForEltwiseAdd(0, abi.Quant(1.0, 0, abi.DT_U8), abi.Quant(1.0, 0, abi.DT_U8),
                                   abi.Quant(1.0, 3, abi.DT_U8), abi.POSTOP_NONE, 0, 0, C.byref(p)) == abi.SUCCESS
    assert (p.mode, p.has_in_mult, p.quant_mult, p.quant_shift, p.clamp_low, p.clamp_high, p.clamp_domain) == \
        (abi.PPE_ADD, 0, 16384, 14, -3, 252, abi.CLAMP_PRE_ZP)


DTYPES = {"u8": abi.DT_U8, "i8": abi.DT_I8, "f16": abi.DT_F16, "bf16": abi.DT_BF16}


@pytest.mark.parametrize("k", KATS["fuse_clamp_37xx"], ids=lambda k: k["name"])
def test_fuse_clamp_lit_cases(k):
    """ncePpeFuseClamp (and the oracle's quantized twin) against the before / after PPE attributes of the reference's
    fuse_clamp lit file."""
    lib = abi.load_library()
    p = abi.PpeTask()
    p.mode, p.clamp_low, p.clamp_high, p.lrelu_mult, p.lrelu_shift = MODES[k["in"]["mode"]], k["in"]["low"], k["in"]["high"], 1024, 13
    rc = lib.ncePpeFuseClamp(abi.Quant(k["scale"], k["zp"], DTYPES[k["dtype"]]), k["min"], k["max"], C.byref(p))
    if k["out"] is None:
        assert rc == abi.ERROR_UNSUPPORTED
        assert (p.mode, p.clamp_low, p.clamp_high) == (MODES[k["in"]["mode"]], k["in"]["low"], k["in"]["high"])
        return
    assert rc == abi.SUCCESS
    assert (p.mode, p.clamp_low, p.clamp_high, p.lrelu_mult, p.lrelu_shift) == (MODES[k["out"]["mode"]], k["out"]["low"], k["out"]["high"], 1024, 13)
    if k["dtype"] in ("u8", "i8"):
        lo, hi = C.c_int32(k["in"]["low"]), C.c_int32(k["in"]["high"])
        assert O.lib().nce_oracle_fuse_clamp_quant(k["scale"], k["zp"], k["min"], k["max"], C.byref(lo), C.byref(hi)) == 0
        assert (lo.value, hi.value) == (k["out"]["low"], k["out"]["high"])


def test_fuse_clamp_float_bits_and_errors():
    """Half and bfloat16 bit patterns against numpy / exact powers of two; range errors."""
    lib = abi.load_library()
    for v in [0.0, 1.0, 6.0, 120.0, 128.0, 65504.0, 1e-3, 0.333251953125, 5.960464477539063e-08, 70000.0, 2049.0, 2051.0]:
        p = abi.PpeTask()
        p.clamp_low, p.clamp_high = -2**31, 2**31 - 1
        assert lib.ncePpeFuseClamp(abi.Quant(1.0, 0, abi.DT_F16), 0.0, v, C.byref(p)) == abi.SUCCESS
        with np.errstate(over="ignore"):
            assert p.clamp_high == int(np.array([v], dtype=np.float32).astype(np.float16).view(np.int16)[0]), v
        assert (p.clamp_low, p.mode) == (-2**31, abi.PPE_LRELUX)
    for v, bits in [(1.0, 0x3F80), (128.0, 0x4300), (6.0, 0x40C0), (1.00390625, 0x3F80), (1.01171875, 0x3F82)]:  # ties to even
        p = abi.PpeTask()
        p.clamp_low, p.clamp_high = -2**31, 2**31 - 1
        assert lib.ncePpeFuseClamp(abi.Quant(1.0, 0, abi.DT_BF16), 0.0, v, C.byref(p)) == abi.SUCCESS
        assert p.clamp_high == bits, v
    p = abi.PpeTask()
    assert lib.ncePpeFuseClamp(abi.Quant(1e-12, 0, abi.DT_U8), 0.0, 1e3, C.byref(p)) == abi.ERROR_INVALID_ARGUMENT  # beyond int32
    assert lib.ncePpeFuseClamp(abi.Quant(0.0, 0, abi.DT_U8), 0.0, 1.0, C.byref(p)) == abi.ERROR_INVALID_ARGUMENT
    assert lib.ncePpeFuseClamp(abi.Quant(1.0, 0, abi.DT_SI32), 0.0, 1.0, C.byref(p)) == abi.ERROR_INVALID_ARGUMENT


def test_weight_set_padding_layout():
    lib = abi.load_library()
    for k in KATS["weights_zero_pad"]:
        sb, pb = C.c_int64(), C.c_int64()
        assert lib.nceConvWeightSetBytes(k["ic"], k["ky"], k["kx"], C.byref(sb), C.byref(pb)) == abi.SUCCESS
        assert [k["oc"], 1, 1, sb.value] == k["padded_shape"] and pb.value == k["pad"]
    sb, pb = C.c_int64(), C.c_int64()
    assert lib.nceConvWeightSetBytes(64, 3, 3, C.byref(sb), C.byref(pb)) == abi.SUCCESS and (sb.value, pb.value) == (576, 0)
    assert lib.nceConvWeightSetBytes(0, 3, 3, C.byref(sb), C.byref(pb)) == abi.ERROR_INVALID_ARGUMENT


def test_weights_table_pointer_contract():
    """Words [0] and [1]: the generator's tables pass; re-ordered pointers, a misaligned step and a sparsity pointer do not."""
    lib = abi.load_library()
    oc = 8
    t = (C.c_int32 * (4 * oc))()
    ws = (C.c_double * 1)(0.01)
    assert lib.nceWeightsTableFill(1, oc, 4096, 576, 0xFFFFFF, 0.02, 0.05, ws, 1, None, t) == abi.SUCCESS
    assert lib.nceWeightsTableCheck(t, oc, 576) == abi.SUCCESS
    t[4 * 3], t[4 * 4] = t[4 * 4], t[4 * 3]
    assert lib.nceWeightsTableCheck(t, oc, 576) == abi.ERROR_UNSUPPORTED
    t[4 * 3], t[4 * 4] = t[4 * 4], t[4 * 3]
    t[4 * 2 + 1] = 1024
    assert lib.nceWeightsTableCheck(t, oc, 576) == abi.ERROR_UNSUPPORTED
    t[4 * 2 + 1] = 0xFFFFFF
    assert lib.nceWeightsTableCheck(t, oc, 568) == abi.ERROR_INVALID_ARGUMENT
    assert lib.nceWeightsTableCheck(t, oc, 592) == abi.ERROR_UNSUPPORTED


def test_ppe_register_field_widths(validator):
    """The validator accepts every PPE field at the largest value its register field holds (the masks of the reference's
    register-map unit test) and rejects the next value."""
    import npu_plugin_amd as nce
    from tests import cases as K
    m = KATS["ppe_register_field_masks_37xx"]

    def rc(case):
        task = K.build_task(case, case.input, case.weights, case.table, np.zeros(case.out_shape, dtype=np.uint8))
        return validator.validate_code(task)

    ok = lambda **ppe: K.conv_case(1, 1, 4, 4, 16, 16, ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, **ppe))
    assert rc(ok(lrelu_mult=m["ppe_prelu_mult"], lrelu_shift=m["ppe_prelu_shift"])) == abi.SUCCESS
    assert rc(ok(lrelu_mult=m["ppe_prelu_mult"] + 1, lrelu_shift=0)) == abi.ERROR_INVALID_ARGUMENT
    assert rc(ok(lrelu_mult=1, lrelu_shift=m["ppe_prelu_shift"] + 1)) == abi.ERROR_INVALID_ARGUMENT
    e = lambda **kw: K.eltwise_case(2, 1, 4, 4, 16, **kw)
    assert rc(e(mult=m["ppe_scale_mult"], shift=m["ppe_scale_shift"], in1_mult=m["elop_scale_a"], in2_mult=m["elop_scale_b"])) == abi.SUCCESS
    assert rc(e(mult=m["ppe_scale_mult"] + 1)) == abi.ERROR_INVALID_ARGUMENT
    assert rc(e(shift=m["ppe_scale_shift"] + 1)) == abi.ERROR_INVALID_ARGUMENT
    assert rc(e(in1_mult=m["elop_scale_a"] + 1)) == abi.ERROR_INVALID_ARGUMENT
    assert rc(e(in2_mult=m["elop_scale_b"] + 1)) == abi.ERROR_INVALID_ARGUMENT
    assert rc(e(ppe_extra=dict(round_mode=m["ppe_scale_round"]))) == abi.ERROR_INVALID_ARGUMENT  # three modes: 0..2
    # the 9-bit zero-point register holds every u8 and i8 zero point
    assert m["ppe_g8_bias_c"] >= 255 and -(m["ppe_g8_bias_c"] + 1) // 2 <= -128
    # table word [2]: shift in 6 bits at bit 8, multiplier in 16 bits at bit 16
    w = O.lib().nce_oracle_scale_word(1, m["ppe_scale_shift"], m["ppe_scale_mult"], 1) & 0xFFFFFFFF
    assert w == (m["ppe_scale_mult"] << 16) | (m["ppe_scale_shift"] << 8)
