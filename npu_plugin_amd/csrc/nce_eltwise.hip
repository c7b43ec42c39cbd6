// ELTWISE add task: out = PPE(in1_mult * (a - zp_a) + in2_mult * (b - zp_b)).
// Semantics: src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:1541-1555
// (per-input multipliers elop_scale_a/b) and :1651-1757 (scale override from the PPE task).
//
// Memory-bound: each lane moves one 16-byte channel group of both inputs and of the output
// (global_load_dwordx4 x2, global_store_dwordx4 x1), 48 algorithmic bytes per 16 outputs. The
// requantize runs in FP64 (exact, see nce_ppe_device.h); per-channel tables and shifts above 52
// take the integer path.
#include "nce_conv_common.h"

namespace nce {
namespace {

template <bool SIGNED>
__device__ __forceinline__ int32_t byte_at(uint32_t w, int i) {
    return SIGNED ? (int32_t)(int8_t)(w >> (8 * i)) : (int32_t)((w >> (8 * i)) & 0xFFu);
}

struct EltArgs {
    TaskDev t;
    Box box;
    int64_t nchunks;
    double M, B;  // uniform scale constants (no weight table)
    int32_t c0;   // -(in1_mult * zp_a + in2_mult * zp_b)
    int32_t may_sat;
    // folded path: outputs are computed as bytes 0..255 (signed outputs 128 higher, flipped back by an XOR on
    // the packed word; B carries the output zero point and that 128), clamp bounds in that domain
    int32_t ilo, ihi;
    uint32_t flip;
    // high-word path: the folded path in integers. y = high word of acc * mq + cq with mq = quant_mult * 2^(32 - shift)
    // and cq = (2^(shift-1) + zero point * 2^shift) * 2^(32 - shift); acc = in1_mult * a + in2_mult * b + c0h as one
    // unsigned 16-bit dot product (signed inputs enter 128 higher, c0h takes that back).
    int32_t mq, c0h;
    int64_t cq;
    uint32_t mults;     // in1_mult | in2_mult << 16
    uint32_t in_flip;   // 0x80808080 for signed inputs
};

// PATH = a PPE_MODE_* value with uniform scale, PATH_TABLE: integer with a per-channel table, or PATH_HI.
constexpr int PATH_TABLE = 4;
constexpr int PATH_HI = 5;
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

template <bool FLAT, int PATH, bool SIGNED>
__global__ __launch_bounds__(256) void eltwise_kernel(EltArgs a) {
    prefetch_kernel_arguments<sizeof(EltArgs)>();
    const TaskDev& t = a.t;
    const Box& box = a.box;
    const int32_t cgroups = box.bc >> 4;
    const PpeF64 pu = ppe_f64_setup(t.ppe, a.may_sat != 0);
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < a.nchunks;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t off_a, off_b, off_o;
        int32_t oc = 0;
        if (FLAT) {
            off_a = off_b = off_o = idx << 4;
            if (PATH == PATH_TABLE) oc = (int32_t)(idx % cgroups) << 4;
        } else {
            int64_t r = idx;
            const int32_t cg = (int32_t)(r % cgroups);
            r /= cgroups;
            const int32_t bx = (int32_t)(r % box.bw);
            r /= box.bw;
            const int32_t by = (int32_t)(r % box.bh);
            const int64_t n = r / box.bh;
            oc = box.z0 + (cg << 4);
            const int64_t y = box.y0 + by, x = box.x0 + bx;
            off_a = n * t.in.sn + y * t.in.sh + x * t.in.sw + oc;
            off_b = n * t.in2.sn + y * t.in2.sh + x * t.in2.sw + oc;
            off_o = n * t.out.sn + y * t.out.sh + x * t.out.sw + oc * t.out.sc;
        }
        const uint4 va = *reinterpret_cast<const uint4*>(t.in.data + off_a);
        const uint4 vb = *reinterpret_cast<const uint4*>(t.in2.data + off_b);
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w};
        const uint32_t wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t wo[4];
        if (PATH == PATH_HI) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t ua = SIGNED ? wa[d] ^ 0x80808080u : wa[d], ub = SIGNED ? wb[d] ^ 0x80808080u : wb[d];
                uint32_t packed = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // bytes i of a and b, zero-extended to a pair of 16-bit values: 0x0c selects a zero byte
                    const uint32_t pair = __builtin_amdgcn_perm(ub, ua, 0x0c040c00u + (uint32_t)i * 0x00010001u);
                    const int32_t acc = (int32_t)__builtin_amdgcn_udot2(__builtin_bit_cast(u16x2, pair), __builtin_bit_cast(u16x2, a.mults),
                                                                         (uint32_t)a.c0h, false);
                    const int32_t y = clamp_med3((int32_t)(((int64_t)acc * a.mq + a.cq) >> 32), a.ilo, a.ihi);
                    packed = i == 0 ? (uint32_t)y : (packed | ((uint32_t)y << (8 * i)));
                }
                wo[d] = packed ^ a.flip;
            }
        } else
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t packed = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // |acc| < 2^26: 16-bit multipliers times 9-bit values, twice, plus c0
                const int32_t acc = t.ppe.in1_mult * byte_at<SIGNED>(wa[d], i) + t.ppe.in2_mult * byte_at<SIGNED>(wb[d], i) + a.c0;
                int32_t y;
                if (PATH == PPE_MODE_FOLDED) {
                    // The conversion truncates; below zero that differs from floor, but every value below zero
                    // clamps to a.ilo >= 0 either way.
                    y = clamp_med3((int32_t)__builtin_fma((double)acc, a.M, a.B), a.ilo, a.ihi);
                } else if (PATH < PPE_MODE_INT) {
                    y = ppe_finish_mode<PATH>(__builtin_fma((double)acc, a.M, a.B), pu);
                } else if (PATH == PPE_MODE_INT) {
                    y = ppe_apply(acc, 0, t.ppe.quant_mult, t.ppe.quant_shift, t.ppe);
                } else {
                    const int32_t* row = t.table + (int64_t)(oc + 4 * d + i) * t.table_stride;
                    y = ppe_apply(acc, row[3], table_mult(row[2]), table_shift(row[2]), t.ppe);
                }
                packed = i == 0 ? ((uint32_t)y & 0xFFu) : (packed | (((uint32_t)y & 0xFFu) << (8 * i)));
            }
            wo[d] = PATH == PPE_MODE_FOLDED ? packed ^ a.flip : packed;
        }
        store_channels16(t.out.data + off_o, FLAT ? 1 : t.out.sc, wo[0], wo[1], wo[2], wo[3]);
    }
}

bool is_dense_nhwc(const TensorDev& x) {
    return x.sc == 1 && x.sw == x.c && x.sh == (int64_t)x.w * x.c && x.sn == (int64_t)x.h * x.w * x.c;
}

template <bool FLAT, int PATH>
hipError_t launch_signed(const EltArgs& a, int grid, hipStream_t s) {
    if (a.t.in.is_signed) return emit(eltwise_kernel<FLAT, PATH, true>, dim3(grid), dim3(256), 0, s, a);
    return emit(eltwise_kernel<FLAT, PATH, false>, dim3(grid), dim3(256), 0, s, a);
}

template <bool FLAT>
hipError_t launch_path(const EltArgs& a, int path, int grid, hipStream_t s) {
    if (path == PPE_MODE_FOLDED) return launch_signed<FLAT, PPE_MODE_FOLDED>(a, grid, s);
    if (path == PPE_MODE_SLOPE) return launch_signed<FLAT, PPE_MODE_SLOPE>(a, grid, s);
    if (path == PPE_MODE_INT) return launch_signed<FLAT, PPE_MODE_INT>(a, grid, s);
    if (path == PATH_HI) return launch_signed<FLAT, PATH_HI>(a, grid, s);
    return launch_signed<FLAT, PATH_TABLE>(a, grid, s);
}


// Fills the launch arguments and returns the arithmetic path (a PPE_MODE_* value, PATH_TABLE or PATH_HI).
static int prepare(const TaskDev& t, EltArgs& a) {
    a.t = t;
    a.c0 = -(t.ppe.in1_mult * t.in.zp + t.ppe.in2_mult * t.in2.zp);
    const int shift = t.ppe.quant_shift;
    a.M = ldexp((double)t.ppe.quant_mult, -shift);
    a.B = (t.ppe.round_mode == NCE_ROUND_HALF_UP && shift > 0) ? 0.5 : 0.0;
    a.may_sat = ppe_may_saturate(((int64_t)t.ppe.in1_mult + t.ppe.in2_mult) * 255, 0, t.ppe.quant_mult, shift);
    // the same selection the table-driven kernels make per workgroup, made here on the host
    const bool half_up = t.ppe.round_mode == NCE_ROUND_HALF_UP;
    const bool prelu = !(t.ppe.prelu_mult == 1 && t.ppe.prelu_shift == 0);
    const int64_t am = t.ppe.prelu_mult < 0 ? -(int64_t)t.ppe.prelu_mult : (int64_t)t.ppe.prelu_mult;
    const bool prelu_sat = am > ((int64_t)1 << t.ppe.prelu_shift);
    int path;
    if (t.table != nullptr) path = PATH_TABLE;
    else if (shift > kMaxF64Shift || !half_up || a.may_sat || (prelu && prelu_sat)) path = PPE_MODE_INT;
    else path = prelu ? PPE_MODE_SLOPE : PPE_MODE_FOLDED;
    a.ilo = a.ihi = 0;
    a.flip = 0;
    a.mq = a.c0h = 0;
    a.cq = 0;
    a.mults = a.in_flip = 0;
    if (path == PPE_MODE_FOLDED) {
        const int32_t lo_zp = t.ppe.lo + t.ppe.zp_out, hi_zp = t.ppe.hi + t.ppe.zp_out;
        const int32_t sb = lo_zp < 0 ? 128 : 0;  // only signed storage clamps below zero
        a.B += (double)(t.ppe.zp_out + sb);
        a.ilo = lo_zp + sb;
        a.ihi = hi_zp + sb;
        a.flip = sb ? 0x80808080u : 0u;
        // The integer form of the same: multiplier scaled to 2^32 must fit int32, input multipliers 16 bits.
        const int64_t mq = (shift >= 1 && shift <= 32) ? (int64_t)t.ppe.quant_mult << (32 - shift) : -1;
        if (mq >= 0 && mq <= 0x7fffffffLL && t.ppe.in1_mult >= 0 && t.ppe.in1_mult <= 65535 && t.ppe.in2_mult >= 0 &&
            t.ppe.in2_mult <= 65535) {
            path = PATH_HI;
            a.mq = (int32_t)mq;
            a.cq = (((int64_t)1 << (shift - 1)) << (32 - shift)) + ((int64_t)(t.ppe.zp_out + sb) << 32);
            a.mults = (uint32_t)t.ppe.in1_mult | ((uint32_t)t.ppe.in2_mult << 16);
            a.in_flip = t.in.is_signed ? 0x80808080u : 0u;
            a.c0h = a.c0 - (t.in.is_signed ? 128 * (t.ppe.in1_mult + t.ppe.in2_mult) : 0);
        }
    }
    return path;
}

}  // namespace

bool eltwise_fuse_params(const TaskDev& add, bool produced_is_in1, FuseAdd* out) {
    EltArgs a;
    if (prepare(add, a) != PATH_HI || add.in.is_signed != add.in2.is_signed) return false;
    out->mults = produced_is_in1 ? a.mults : ((a.mults >> 16) | (a.mults << 16));
    out->in_flip = a.in_flip;
    out->c0h = a.c0h;
    out->mq = a.mq;
    out->cq = a.cq;
    out->ilo = a.ilo;
    out->ihi = a.ihi;
    out->flip = a.flip;
    return true;
}

hipError_t launch_eltwise(const TaskDev& t, const Box& box, hipStream_t stream) {
    EltArgs a;
    a.box = box;
    a.nchunks = (int64_t)t.out.n * box.bh * box.bw * (box.bc >> 4);
    if (a.nchunks == 0) return hipSuccess;
    const bool full = box.x0 == 0 && box.y0 == 0 && box.z0 == 0 && box.bw == t.out.w && box.bh == t.out.h &&
                      box.bc == t.out.c;
    const bool flat = full && is_dense_nhwc(t.in) && is_dense_nhwc(t.in2) && is_dense_nhwc(t.out);
    const int path = prepare(t, a);
    int64_t blocks = (a.nchunks + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    return flat ? launch_path<true>(a, path, (int)blocks, stream) : launch_path<false>(a, path, (int)blocks, stream);
}

}  // namespace nce
