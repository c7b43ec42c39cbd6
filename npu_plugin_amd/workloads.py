"""Synthetic NCE task workloads (the benchmark configurations and the generators behind them).

A case holds host (numpy) tensors and the attributes of one task. `build_task` turns it into an
NCEClusterTask over any set of buffers (numpy for the oracle, torch.cuda for the HIP executor), so both
sides consume the very same descriptor content.
"""
import math
from dataclasses import dataclass, field

import numpy as np

from . import nce_task as nce


def approx(bits, target):
    """mult/shift pair for synthetic tables (frexp split with truncated mantissa)."""
    m, e = math.frexp(target)
    return int(m * 2 ** bits), bits - e


def make_table(rng, oc, w_step, scale_lo=1e-3, scale_hi=1e-2, bias_sigma=1000.0, ptr_base=0):
    """Weight table rows {ptr, 0xFFFFFF, (mult<<16)|(shift<<8), bias} with per-channel random scales."""
    t = np.zeros((oc, 4), dtype=np.int64)
    scales = rng.uniform(scale_lo, scale_hi, size=oc)
    for c in range(oc):
        m, s = approx(15, float(scales[c]))
        assert 0 <= s <= 63 and 0 <= m <= 65535
        t[c, 0] = ptr_base + c * w_step
        t[c, 1] = 0xFFFFFF
        t[c, 2] = (m << 16) | (s << 8)
        t[c, 3] = int(round(rng.normal(0.0, bias_sigma)))
    return (t & 0xFFFFFFFF).astype(np.uint32).view(np.int32).reshape(oc, 4).copy()


def _np_dtype(signed):
    return np.int8 if signed else np.uint8


def _rand8(rng, shape, signed, lo=None, hi=None):
    if signed:
        lo = -128 if lo is None else lo
        hi = 127 if hi is None else hi
    else:
        lo = 0 if lo is None else lo
        hi = 255 if hi is None else hi
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int64).astype(_np_dtype(signed))


@dataclass
class Case:
    name: str
    task_type: int
    input: np.ndarray                 # (N, H, W, C)
    out_shape: tuple                  # (N, OH, OW, OC)
    in_zp: int = 0
    out_zp: int = 0
    out_signed: bool = False
    weights: np.ndarray = None        # conv (OC,KY,KX,IC) | dw (C, 16k) | eltwise second input (N,H,W,C)
    w_zp: int = 0
    table: np.ndarray = None          # (OC, 4) int32
    kernel: tuple = None              # (KY, KX)
    strides: tuple = None             # (SY, SX)
    pads: tuple = (0, 0, 0, 0)        # left, right, top, bottom
    ppe: dict = field(default_factory=dict)   # kwargs of addPPETask; empty = no PPE task
    variants: list = None             # list of (outStart, outEnd); None = one whole-output variant

    def ops(self):
        n, oh, ow, oc = self.out_shape
        if self.task_type == nce.TASK_CONV:
            return 2 * n * oh * ow * oc * self.kernel[0] * self.kernel[1] * self.input.shape[3]
        if self.task_type == nce.TASK_DWCONV:
            return 2 * n * oh * ow * oc * self.kernel[0] * self.kernel[1]
        return 0

    def algorithmic_bytes(self):
        b = self.input.nbytes + int(np.prod(self.out_shape))
        if self.weights is not None:
            if self.task_type == nce.TASK_DWCONV:
                b += self.weights.shape[0] * 16 * ((self.kernel[0] * self.kernel[1] + 15) // 16)
            else:
                b += self.weights.nbytes
        if self.table is not None:
            b += self.table.nbytes
        return b


def out_hw(h, w, k, s, pads):
    left, right, top, bottom = pads
    return (h + top + bottom - k[0]) // s[0] + 1, (w + left + right - k[1]) // s[1] + 1


def variant_pad(case, start, end):
    """The part of the kernel padding a sub-box touches (what the compiler stores per DPUTask)."""
    if case.task_type == nce.TASK_ELTWISE:
        return (0, 0, 0, 0)
    left, right, top, bottom = case.pads
    (ky, kx), (sy, sx) = case.kernel, case.strides
    h, w = case.input.shape[1], case.input.shape[2]
    pl = max(0, left - start[0] * sx)
    pt = max(0, top - start[1] * sy)
    pr = max(0, end[0] * sx - left + kx - 1 - (w - 1))
    pb = max(0, end[1] * sy - top + ky - 1 - (h - 1))
    return (pl, pr, pt, pb)


def build_task(case, input, weights, table, output):
    """Buffers may be numpy arrays (host) or torch tensors (device); they must match the case's shapes."""
    kw = {}
    if case.task_type != nce.TASK_ELTWISE:
        kw = dict(kernel_size=list(case.kernel), kernel_strides=list(case.strides), kernel_padding=case.pads)
    w_op = None
    if weights is not None:
        if case.task_type == nce.TASK_CONV:
            w_op = nce.conv_weights(weights, case.w_zp)
        elif case.task_type == nce.TASK_DWCONV:
            w_op = nce.depthwise_weights(weights, case.w_zp)
        else:
            w_op = nce.activation(weights, case.w_zp)
    task = nce.NCEClusterTask(case.task_type, nce.activation(input, case.in_zp), w_op,
                              nce.weight_table(table) if table is not None else None,
                              nce.activation(output, case.out_zp), **kw)
    if case.variants is None:
        task.addWholeOutputDPUTask()
    else:
        for start, end in case.variants:
            task.addDPUTask(list(start), list(end), variant_pad(case, start, end))
    if case.ppe:
        task.addPPETask(**case.ppe)
    return task


class DeviceCase:
    """The case's tensors resident on the GPU + the task over them."""

    def __init__(self, case, device="cuda:0"):
        import torch
        self.case = case
        self.input = torch.from_numpy(case.input).to(device)
        self.weights = torch.from_numpy(case.weights).to(device) if case.weights is not None else None
        self.table = torch.from_numpy(case.table).to(device) if case.table is not None else None
        self.output = torch.zeros(case.out_shape, dtype=torch.int8 if case.out_signed else torch.uint8, device=device)
        self.task = build_task(case, self.input, self.weights, self.table, self.output)


def run_hip(case, executor):
    import torch
    dc = DeviceCase(case)
    dc.output.fill_(0x5A if not case.out_signed else 0x5A - 128)  # poison: untouched bytes must not look right
    stream = torch.cuda.current_stream().cuda_stream
    executor.enqueue(dc.task, stream)
    executor.synchronize(stream)
    return dc.output.cpu().numpy()


# ------------------------------------------------------------------------------------------------
# generators
# ------------------------------------------------------------------------------------------------

def conv_case(seed, n, h, w, ic, oc, k=(3, 3), s=(1, 1), pads=(1, 1, 1, 1), in_signed=False, w_signed=True, in_zp=128,
              w_zp=0, out_zp=128, out_signed=False, ppe=None, scale_lo=1e-3, scale_hi=1e-2, bias_sigma=1000.0,
              variants=None, name=None):
    rng = np.random.default_rng(seed)
    x = _rand8(rng, (n, h, w, ic), in_signed)
    wt = _rand8(rng, (oc, k[0], k[1], ic), w_signed, lo=-127 if w_signed else None)
    table = make_table(rng, oc, k[0] * k[1] * ic, scale_lo, scale_hi, bias_sigma)
    oh, ow = out_hw(h, w, k, s, pads)
    if ppe is None:
        ppe = dict(mode=nce.PPE_NOOP, clamp_low=-128 if out_signed else 0, clamp_high=127 if out_signed else 255)
    return Case(name or f"conv{k[0]}x{k[1]}_{n}x{h}x{w}x{ic}_{oc}", nce.TASK_CONV, x, (n, oh, ow, oc), in_zp, out_zp,
                out_signed, wt, w_zp, table, tuple(k), tuple(s), tuple(pads), ppe, variants)


def dw_case(seed, n, h, w, c, k=(3, 3), s=(2, 2), pads=(1, 1, 1, 1), in_signed=False, w_signed=True, in_zp=128, w_zp=0,
            out_zp=128, out_signed=False, ppe=None, scale_lo=1e-3, scale_hi=1e-2, variants=None, name=None):
    rng = np.random.default_rng(seed)
    x = _rand8(rng, (n, h, w, c), in_signed)
    taps = k[0] * k[1]
    row = 16 * ((taps + 15) // 16)
    wt = np.zeros((c, row), dtype=_np_dtype(w_signed))
    wt[:, :taps] = _rand8(rng, (c, taps), w_signed, lo=-127 if w_signed else None)
    table = make_table(rng, c, row, scale_lo, scale_hi)
    oh, ow = out_hw(h, w, k, s, pads)
    if ppe is None:
        ppe = dict(mode=nce.PPE_NOOP, clamp_low=-128 if out_signed else 0, clamp_high=127 if out_signed else 255)
    return Case(name or f"dw{k[0]}x{k[1]}_{n}x{h}x{w}x{c}", nce.TASK_DWCONV, x, (n, oh, ow, c), in_zp, out_zp, out_signed,
                wt, w_zp, table, tuple(k), tuple(s), tuple(pads), ppe, variants)


def pool_case(seed, is_max, n, h, w, c, k=(3, 3), s=(2, 2), pads=(1, 1, 1, 1), in_signed=False, in_zp=128, out_zp=128,
              with_table=False, ppe=None, variants=None, name=None):
    rng = np.random.default_rng(seed)
    x = _rand8(rng, (n, h, w, c), in_signed)
    oh, ow = out_hw(h, w, k, s, pads)
    lo, hi = (-128, 127) if in_signed else (0, 255)
    table = None
    if ppe is None:
        if is_max:
            ppe = dict(mode=nce.PPE_NOOP, clamp_low=lo, clamp_high=hi)
        else:
            m, sh = approx(15, 1.0 / (k[0] * k[1]))
            ppe = dict(mode=nce.PPE_NOOP, clamp_low=lo, clamp_high=hi, quant_mult=m, quant_shift=sh)
    if with_table and not is_max:
        table = make_table(rng, c, 0, 0.5 / (k[0] * k[1]), 2.0 / (k[0] * k[1]), 4.0)
    return Case(name or f"{'max' if is_max else 'avg'}pool{k[0]}x{k[1]}_{n}x{h}x{w}x{c}",
                nce.TASK_MAXPOOL if is_max else nce.TASK_AVEPOOL, x, (n, oh, ow, c), in_zp, out_zp, in_signed, None, 0,
                table, tuple(k), tuple(s), tuple(pads), ppe, variants)


def eltwise_case(seed, n, h, w, c, signed=False, zp_a=120, zp_b=130, out_zp=128, in1_mult=20971, in2_mult=31457,
                 mult=25600, shift=30, with_in_mult=True, with_table=False, ppe_extra=None, variants=None, name=None):
    rng = np.random.default_rng(seed)
    a = _rand8(rng, (n, h, w, c), signed)
    b = _rand8(rng, (n, h, w, c), signed)
    lo, hi = (-128, 127) if signed else (0, 255)
    ppe = dict(mode=nce.PPE_ADD, clamp_low=lo, clamp_high=hi, quant_mult=mult, quant_shift=shift)
    if with_in_mult:
        ppe.update(in1_quant_mult=in1_mult, in2_quant_mult=in2_mult)
    if ppe_extra:
        ppe.update(ppe_extra)
    table = make_table(rng, c, 0, 0.2, 0.9, 8.0) if with_table else None
    return Case(name or f"eltwise_{n}x{h}x{w}x{c}", nce.TASK_ELTWISE, a, (n, h, w, c), zp_a, out_zp, signed, b, zp_b, table,
                None, None, (0, 0, 0, 0), ppe, variants)


# ------------------------------------------------------------------------------------------------
# the benchmark configurations
# ------------------------------------------------------------------------------------------------

SEED = 0x5EED0000


def cfg1():
    return conv_case(SEED + 1, 1, 32, 32, 16, 16, name="cfg1_conv3x3_1x32x32x16_16")


def cfg2(n=8):
    return conv_case(SEED + 2, n, 56, 56, 64, 64, name=f"cfg2_conv3x3_{n}x56x56x64_64_lrelu",
                     ppe=dict(mode=nce.PPE_LPRELU, clamp_low=0, clamp_high=255, lrelu_mult=1638, lrelu_shift=14))


def cfg3_dw(n=16):
    return dw_case(SEED + 3, n, 112, 112, 96, name=f"cfg3_dw3x3s2_{n}x112x112x96")


def cfg3_maxpool(n=16, x=None):
    c = pool_case(SEED + 4, True, n, 56, 56, 96, name=f"cfg3_maxpool3x3s2_{n}x56x56x96")
    if x is not None:
        c.input = x
    return c


def cfg3_avgpool(n=16, x=None):
    c = pool_case(SEED + 5, False, n, 28, 28, 96, k=(2, 2), s=(2, 2), pads=(0, 0, 0, 0),
                  name=f"cfg3_avgpool2x2_{n}x28x28x96")
    if x is not None:
        c.input = x
    return c


def cfg4(n=16):
    return eltwise_case(SEED + 6, n, 28, 28, 256, name=f"cfg4_eltwise_{n}x28x28x256")


# ------------------------------------------------------------------------------------------------
# cfg5: synthetic INT8 ResNet-50 (v1.5) chained through the NCE op path
# ------------------------------------------------------------------------------------------------

@dataclass
class GraphLayer:
    name: str
    task_type: int
    src: int                      # index of the input tensor in the graph's tensor list
    src2: int = -1                # second input (eltwise)
    dst: int = -1
    weights: np.ndarray = None
    table: np.ndarray = None
    kernel: tuple = None
    strides: tuple = None
    pads: tuple = (0, 0, 0, 0)
    ppe: dict = field(default_factory=dict)
    real_ic: int = 0              # un-padded input channels (conv1), for the op count


class ResNet50Graph:
    """53 convolutions (1x1 / 3x3 / 7x7, strides 1 / 2), the 3x3 s2 max pool after conv1 and the 16
    residual adds of ResNet-50 v1.5, all u8 NHWC with zero point 128, random i8 weights and random
    per-channel mult/shift tables. ReLU is the 37XX form: mode NOOP, clamp [zp, 255]."""

    ZP = 128

    def __init__(self, batch=32, size=224, seed=SEED + 7):
        self.batch, self.size = batch, size
        self.rng = np.random.default_rng(seed)
        self.tensors = []   # shapes (N, H, W, C)
        self.layers = []
        x = self._tensor(size, size, 16)      # 3 real channels padded to 16 (zero weights on the padding)
        x = self._conv("conv1", x, 64, (7, 7), (2, 2), (3, 3, 3, 3), relu=True, real_ic=3)
        x = self._maxpool("pool1", x)
        inplanes = 64
        for li, (planes, blocks, stride) in enumerate([(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)], 1):
            for b in range(blocks):
                s = stride if b == 0 else 1
                name = f"layer{li}.{b}"
                y = self._conv(name + ".conv1", x, planes, (1, 1), (1, 1), (0, 0, 0, 0), relu=True)
                y = self._conv(name + ".conv2", y, planes, (3, 3), (s, s), (1, 1, 1, 1), relu=True)
                y = self._conv(name + ".conv3", y, planes * 4, (1, 1), (1, 1), (0, 0, 0, 0), relu=False)
                if b == 0:
                    idt = self._conv(name + ".downsample", x, planes * 4, (1, 1), (s, s), (0, 0, 0, 0), relu=False)
                else:
                    idt = x
                x = self._add(name + ".add", y, idt)
                inplanes = planes * 4
        self.output = x

    # -- construction helpers --------------------------------------------------------------------
    def _tensor(self, h, w, c):
        self.tensors.append((self.batch, h, w, c))
        return len(self.tensors) - 1

    def _conv(self, name, src, oc, k, s, pads, relu, real_ic=0):
        _, h, w, ic = self.tensors[src]
        wt = self.rng.integers(-127, 128, size=(oc, k[0], k[1], ic), dtype=np.int64).astype(np.int8)
        if real_ic:
            wt[:, :, :, real_ic:] = 0
        # Keep activations alive through 50 layers: aim every conv at a pre-activation spread of ~40
        # quantization steps. Inputs are post-ReLU (rms ~ 40 / sqrt(2)) except the image (uniform bytes).
        kk = k[0] * k[1] * (real_ic or ic)
        in_rms = 73.9 if real_ic else 40.0 / math.sqrt(2.0)
        base = 40.0 / (math.sqrt(kk) * in_rms * 73.3)
        table = make_table(self.rng, oc, k[0] * k[1] * ic, 0.85 * base, 1.15 * base, bias_sigma=5.0 / base)
        oh, ow = out_hw(h, w, k, s, pads)
        dst = self._tensor(oh, ow, oc)
        ppe = dict(mode=nce.PPE_NOOP, clamp_low=self.ZP if relu else 0, clamp_high=255)
        self.layers.append(GraphLayer(name, nce.TASK_CONV, src, -1, dst, wt, table, tuple(k), tuple(s), tuple(pads), ppe,
                                      real_ic or ic))
        return dst

    def _maxpool(self, name, src):
        _, h, w, c = self.tensors[src]
        oh, ow = out_hw(h, w, (3, 3), (2, 2), (1, 1, 1, 1))
        dst = self._tensor(oh, ow, c)
        self.layers.append(GraphLayer(name, nce.TASK_MAXPOOL, src, -1, dst, None, None, (3, 3), (2, 2), (1, 1, 1, 1),
                                      dict(mode=nce.PPE_NOOP, clamp_low=0, clamp_high=255)))
        return dst

    def _add(self, name, a, b):
        _, h, w, c = self.tensors[a]
        dst = self._tensor(h, w, c)
        # (a + b) / sqrt(2), ReLU: both inputs x 16384 (shift 14 folded into the output shift)
        ppe = dict(mode=nce.PPE_NOOP, clamp_low=self.ZP, clamp_high=255, quant_mult=23170, quant_shift=29,
                   in1_quant_mult=16384, in2_quant_mult=16384)
        self.layers.append(GraphLayer(name, nce.TASK_ELTWISE, a, b, dst, None, None, None, None, (0, 0, 0, 0), ppe))
        return dst

    # -- accounting ------------------------------------------------------------------------------
    def conv_ops(self):
        total = 0
        for L in self.layers:
            if L.task_type == nce.TASK_CONV:
                n, oh, ow, oc = self.tensors[L.dst]
                total += 2 * n * oh * ow * oc * L.kernel[0] * L.kernel[1] * L.real_ic
        return total

    def layer_bytes(self, L):
        b = int(np.prod(self.tensors[L.src])) + int(np.prod(self.tensors[L.dst]))
        if L.src2 >= 0:
            b += int(np.prod(self.tensors[L.src2]))
        if L.weights is not None:
            b += L.weights.nbytes + L.table.nbytes
        return b

    def make_input(self):
        x = self.rng.integers(0, 256, size=self.tensors[0], dtype=np.int64).astype(np.uint8)
        return x

    # -- task construction over any buffers (numpy or torch) -----------------------------------
    def layer_case(self, L):
        """A Case view of one layer (tensors filled in by the caller)."""
        return Case(L.name, L.task_type, np.empty(0, dtype=np.uint8), self.tensors[L.dst], self.ZP, self.ZP, False, None, 0,
                    None, L.kernel, L.strides, L.pads, L.ppe, None)

    def build_tasks(self, buffers, weights, tables):
        """buffers[i]: activation tensor i; weights/tables[j]: operands of layer j (None where absent)."""
        tasks = []
        for j, L in enumerate(self.layers):
            case = self.layer_case(L)
            case.input = buffers[L.src]            # only shapes/strides/addresses are read
            if L.task_type == nce.TASK_ELTWISE:
                case.w_zp = self.ZP
                tasks.append(build_task(case, buffers[L.src], buffers[L.src2], None, buffers[L.dst]))
            else:
                tasks.append(build_task(case, buffers[L.src], weights[j], tables[j], buffers[L.dst]))
        return tasks


class DeviceGraph:
    """A ResNet50Graph resident on the GPU: activations, weights, tables and one task list."""

    def __init__(self, graph, executor, x=None, device="cuda:0"):
        import torch
        self.graph = graph
        self.buffers = [torch.zeros(s, dtype=torch.uint8, device=device) for s in graph.tensors]
        if x is not None:
            self.buffers[0].copy_(torch.from_numpy(x))
        self.weights = [torch.from_numpy(L.weights).to(device) if L.weights is not None else None for L in graph.layers]
        self.tables = [torch.from_numpy(L.table).to(device) if L.table is not None else None for L in graph.layers]
        self.tasks = graph.build_tasks(self.buffers, self.weights, self.tables)
        self.task_list = executor.task_list()
        for t in self.tasks:
            self.task_list.append(t)

    def run(self, stream):
        self.task_list.enqueue(stream)
