// Fixed-point parameter generation behind include/nce_params.h (host arithmetic only).
// Each routine states the reference function it reproduces; paths are relative to the
// reference's src/vpux_compiler/src/.
#include <cfloat>
#include <climits>
#include <algorithm>
#include <cmath>
#include <cstring>

#include "../../include/nce_params.h"

namespace {

struct Approx {
    int64_t mult;
    int shift;
    int post_shift;
};

// utils/quantization.cpp:242-252: frexp split, mantissa truncated into `bits` bits.
Approx approximate(int bits, double target) {
    int e = 0;
    const double m = std::frexp(target, &e);
    Approx r;
    r.mult = static_cast<int64_t>(m * std::ldexp(1.0, bits));
    r.shift = e > bits ? 0 : bits - e;
    r.post_shift = e > bits ? bits - e : 0;
    return r;
}

bool quant15(int arch, double target, Approx* out) {
    const Approx a = approximate(15, target);
    if (a.mult < 0 || a.mult > 0xFFFF || a.shift < 0 || a.shift > 0xFF) return false;
    if (a.post_shift != 0 && arch != NCE_ARCH_VPUX30XX) return false;  // utils/quantization.cpp:260-263
    *out = a;
    return true;
}

void storage_range(int32_t dtype, int64_t* lo, int64_t* hi) {
    *lo = dtype == NCE_DT_U8 ? 0 : -128;
    *hi = dtype == NCE_DT_U8 ? 255 : 127;
}

bool float_equal(float a, float b) {
    return std::fabs(a - b) <= FLT_EPSILON;
}

// Stage 1, utils/VPU/ppe_utils.cpp:293-376: clamps in the zero-point-free domain.
bool stage1(int arch, int postop, double p0, double p1, const nce_quant_t& out, nce_ppe_task_t* ppe, bool* had_postop) {
    int64_t smin, smax;
    storage_range(out.dtype, &smin, &smax);
    const int64_t lo_q = smin - out.zero_point, hi_q = smax - out.zero_point;
    ppe->mode = NCE_PPE_NOOP;
    ppe->clamp_low = static_cast<int32_t>(lo_q);
    ppe->clamp_high = static_cast<int32_t>(hi_q);
    ppe->lrelu_mult = 1;
    ppe->lrelu_shift = 0;
    ppe->clamp_domain = NCE_CLAMP_PRE_ZP;
    *had_postop = postop != NCE_POSTOP_NONE;
    if (postop == NCE_POSTOP_NONE) return true;
    if (postop == NCE_POSTOP_RELU) {
        ppe->mode = NCE_PPE_LRELU;
        ppe->clamp_low = 0;
        return true;
    }
    if (postop == NCE_POSTOP_CLAMP) {  // utils/quantization.cpp:364-380
        const int64_t qmin = std::llround(p0 / out.scale), qmax = std::llround(p1 / out.scale);
        ppe->clamp_low = static_cast<int32_t>(lo_q > qmin ? lo_q : qmin);
        ppe->clamp_high = static_cast<int32_t>(hi_q < qmax ? hi_q : qmax);
        return true;
    }
    if (postop == NCE_POSTOP_LEAKY_RELU) {
        if (arch != NCE_ARCH_VPUX37XX) return false;  // quantized LeakyReLU on 30XX is a PWL table, not this path
        ppe->mode = NCE_PPE_LPRELU;
        const float af = static_cast<float>(p0);
        if (float_equal(af, 0.0f)) {
            ppe->lrelu_mult = 0;
        } else if (!float_equal(af, 1.0f)) {
            const Approx a = approximate(11, p0);  // utils/quantization.cpp:344-354
            if (a.post_shift != 0) return false;
            ppe->lrelu_mult = static_cast<int32_t>(a.mult);
            ppe->lrelu_shift = a.shift;
        }
        return true;
    }
    return false;
}

// Stage 2, dialect/VPU/transforms/passes/setup_ppe.cpp:12-33 and :123-195 (37XX only).
void stage2_37xx(bool has_ppe, const nce_quant_t& out, nce_ppe_task_t* ppe) {
    int64_t smin, smax;
    storage_range(out.dtype, &smin, &smax);
    const int32_t lo = has_ppe ? ppe->clamp_low : INT32_MIN;
    const int32_t hi = has_ppe ? ppe->clamp_high : INT32_MAX;
    const int32_t lm = has_ppe ? ppe->lrelu_mult : 1;
    const int32_t ls = has_ppe ? ppe->lrelu_shift : 0;
    const bool hi_is_max_minus_zp = smax - out.zero_point == hi;
    int32_t mode = NCE_PPE_NOOP;
    if (has_ppe && (lm != 1 || ls != 0)) mode = NCE_PPE_LPRELU;
    else if (hi_is_max_minus_zp && lo == 0) mode = NCE_PPE_NOOP;
    else if ((hi == INT32_MAX || hi == 0) && lo == 0) mode = NCE_PPE_LRELU;
    else if (hi < INT32_MAX && lo == 0) mode = NCE_PPE_LRELUX;
    int64_t nlo, nhi;
    if (mode == NCE_PPE_NOOP) {
        nlo = has_ppe ? static_cast<int64_t>(lo) + out.zero_point : smin;
        nhi = has_ppe ? static_cast<int64_t>(hi) + out.zero_point : smax;
    } else {
        nlo = smin;
        nhi = mode == NCE_PPE_LRELUX ? hi : smax;
    }
    ppe->mode = mode;
    ppe->clamp_low = static_cast<int32_t>(nlo);
    ppe->clamp_high = static_cast<int32_t>(nhi);
    ppe->lrelu_mult = lm;
    ppe->lrelu_shift = ls;
    ppe->clamp_domain = NCE_CLAMP_POST_ZP;
}

void clear_quant(nce_ppe_task_t* ppe) {
    ppe->has_quant = 0;
    ppe->quant_mult = 1;
    ppe->quant_shift = 0;
    ppe->quant_post_shift = 0;
    ppe->has_in_mult = 0;
    ppe->in1_quant_mult = 1;
    ppe->in2_quant_mult = 1;
    ppe->round_mode = NCE_ROUND_HALF_UP;
}

}  // namespace

extern "C" {

nce_result_t nceQuantApproximate(int32_t arch, double target, int32_t* mult, int32_t* shift, int32_t* post_shift) {
    if (!mult || !shift || !post_shift) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    Approx a;
    if (!quant15(arch, target, &a)) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *mult = static_cast<int32_t>(a.mult);
    *shift = a.shift;
    *post_shift = a.post_shift;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceEltwiseQuantApproximate(int32_t arch, double in1_scale, double in2_scale, double out_scale,
                                        int32_t* in1_mult, int32_t* in2_mult, int32_t* out_mult, int32_t* out_shift) {
    if (!in1_mult || !in2_mult || !out_mult || !out_shift) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    Approx a, b, o;
    if (!quant15(arch, in1_scale, &a) || !quant15(arch, in2_scale, &b) || !quant15(arch, 1.0 / out_scale, &o))
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    const int lo = a.shift < b.shift ? a.shift : b.shift;
    const int hi = a.shift > b.shift ? a.shift : b.shift;
    const int64_t reg_shift_max = 63, reg_mult_max = 65535;  // 6-bit shift, 16-bit mult registers
    const bool up = hi + o.shift <= reg_shift_max && a.mult <= (reg_mult_max >> (hi - a.shift)) &&
                    b.mult <= (reg_mult_max >> (hi - b.shift));
    if (up) {
        a.mult = static_cast<uint16_t>(a.mult << (hi - a.shift));
        b.mult = static_cast<uint16_t>(b.mult << (hi - b.shift));
        o.shift = static_cast<uint8_t>(o.shift + hi);
    } else if (lo + o.shift < reg_shift_max) {
        a.mult = static_cast<uint16_t>(a.mult >> (a.shift - lo));
        b.mult = static_cast<uint16_t>(b.mult >> (b.shift - lo));
        o.shift = static_cast<uint8_t>(o.shift + lo);
    } else {
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;  // "out of register range"
    }
    *in1_mult = static_cast<int32_t>(a.mult);
    *in2_mult = static_cast<int32_t>(b.mult);
    *out_mult = static_cast<int32_t>(o.mult);
    *out_shift = o.shift;
    return NCE_RESULT_SUCCESS;
}

nce_result_t ncePReLUApproximate(int32_t arch, double alpha, int32_t* mult, int32_t* shift) {
    if (!mult || !shift) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    const Approx a = approximate(arch == NCE_ARCH_VPUX30XX ? 7 : 11, alpha);
    if (a.post_shift != 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *mult = static_cast<int32_t>(a.mult);
    *shift = a.shift;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceWeightsTableFill(int32_t arch, int32_t oc, int32_t weights_ptr, int32_t weights_ptr_step,
                                 int32_t sparsity_ptr, double in_scale, double out_scale,
                                 const double* weight_scales, int32_t n_weight_scales, const double* bias,
                                 int32_t* table) {
    if (!weight_scales || !table || oc <= 0 || (n_weight_scales != 1 && n_weight_scales != oc))
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    int64_t wptr = weights_ptr;
    for (int32_t c = 0; c < oc; ++c, wptr += weights_ptr_step) {
        if (wptr % 16 != 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;                                // nce_sparsity.cpp:504-506
        if (sparsity_ptr != 0xFFFFFF && sparsity_ptr % 16 != 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;  // :507-510
        const double ws = weight_scales[n_weight_scales == 1 ? 0 : c];
        Approx a;
        if (!quant15(arch, ws * in_scale / out_scale, &a)) return NCE_RESULT_ERROR_INVALID_ARGUMENT;  // :261-264
        uint32_t word2 = (static_cast<uint32_t>(a.shift) << 8) | (static_cast<uint32_t>(a.mult) << 16);  // :141-155
        if (arch == NCE_ARCH_VPUX30XX) word2 |= 1u | (1u << 14);                                       // :122-139
        int32_t b = 0;
        if (bias != nullptr) {  // :186-193, :646-676
            const double v = bias[c] / (ws * in_scale);
            if (v <= static_cast<double>(INT32_MIN) || v >= static_cast<double>(INT32_MAX)) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
            b = static_cast<int32_t>(std::round(v));
        }
        int32_t* row = table + 4 * static_cast<int64_t>(c);
        row[0] = static_cast<int32_t>(wptr);
        row[1] = sparsity_ptr;
        memcpy(&row[2], &word2, 4);
        row[3] = b;
    }
    return NCE_RESULT_SUCCESS;
}

nce_result_t ncePpeFromPostOp(int32_t arch, int32_t postop, double p0, double p1, nce_quant_t out, nce_ppe_task_t* ppe) {
    if (!ppe) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    clear_quant(ppe);
    bool had = false;
    if (!stage1(arch, postop, p0, p1, out, ppe, &had)) return NCE_RESULT_ERROR_UNSUPPORTED;
    if (arch == NCE_ARCH_VPUX37XX) stage2_37xx(had, out, ppe);
    return NCE_RESULT_SUCCESS;
}

nce_result_t ncePpeForAvgPool(int32_t arch, nce_quant_t in, nce_quant_t out, int32_t ky, int32_t kx, int32_t postop,
                              double p0, double p1, nce_ppe_task_t* ppe) {
    if (!ppe || ky <= 0 || kx <= 0 || in.scale == 0 || out.scale == 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    clear_quant(ppe);
    bool had = false;
    if (!stage1(arch, postop, p0, p1, out, ppe, &had)) return NCE_RESULT_ERROR_UNSUPPORTED;
    Approx a;
    if (!quant15(arch, in.scale / out.scale / static_cast<double>(static_cast<int64_t>(ky) * kx), &a))  // ppe_utils.cpp:72-106
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    ppe->has_quant = 1;
    ppe->quant_mult = static_cast<int32_t>(a.mult);
    ppe->quant_shift = a.shift;
    ppe->quant_post_shift = a.post_shift;
    if (arch == NCE_ARCH_VPUX37XX) stage2_37xx(true, out, ppe);  // the op always carries a PPE attribute
    return NCE_RESULT_SUCCESS;
}

nce_result_t ncePpeForEltwiseAdd(int32_t arch, nce_quant_t in1, nce_quant_t in2, nce_quant_t out, int32_t postop,
                                 double p0, double p1, nce_ppe_task_t* ppe) {
    if (!ppe || in1.scale == 0 || in2.scale == 0 || out.scale == 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    clear_quant(ppe);
    bool had = false;
    if (!stage1(arch, postop, p0, p1, out, ppe, &had)) return NCE_RESULT_ERROR_UNSUPPORTED;
    ppe->mode = NCE_PPE_ADD;  // getPPEMode(EltwiseType::ADD): the post-op only supplies clamps and slope
    if (arch == NCE_ARCH_VPUX37XX) {                         // supportsPerInputEltwiseScale
        int32_t m1, m2, mo, so;
        const nce_result_t r = nceEltwiseQuantApproximate(arch, in1.scale, in2.scale, out.scale, &m1, &m2, &mo, &so);
        if (r != NCE_RESULT_SUCCESS) return r;
        ppe->has_quant = 1;
        ppe->quant_mult = mo;
        ppe->quant_shift = so;
        ppe->has_in_mult = 1;
        ppe->in1_quant_mult = m1;
        ppe->in2_quant_mult = m2;
        stage2_37xx(true, out, ppe);
    } else {
        Approx a;  // single scale in1/out: ppe_utils.cpp:18-70
        if (!quant15(arch, in1.scale / out.scale, &a)) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
        ppe->has_quant = 1;
        ppe->quant_mult = static_cast<int32_t>(a.mult);
        ppe->quant_shift = a.shift;
        ppe->quant_post_shift = a.post_shift;
    }
    return NCE_RESULT_SUCCESS;
}

// Bits of a float converted to IEEE half / bfloat16 with round-to-nearest-even, sign-extended from 16 bits
// (the reference reinterprets the 16-bit pattern as int16_t, fuse_clamp.cpp:54-57,63-66).
static int32_t f16_bits(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const int32_t exp = static_cast<int32_t>((x >> 23) & 0xFF) - 127 + 15;
    uint32_t man = x & 0x7FFFFFu;
    uint32_t h;
    if (((x >> 23) & 0xFF) == 0xFF) {
        h = sign | 0x7C00u | (man ? 0x200u : 0u);
    } else if (exp >= 31) {
        h = sign | 0x7C00u;
    } else if (exp <= 0) {
        if (exp < -10) {
            h = sign;
        } else {
            man |= 0x800000u;
            const int shift = 14 - exp;  // 14..24
            uint32_t r = man >> shift;
            const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
            if (rem > half || (rem == half && (r & 1))) ++r;
            h = sign | r;
        }
    } else {
        uint32_t r = (static_cast<uint32_t>(exp) << 10) | (man >> 13);
        const uint32_t rem = man & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) ++r;  // a carry into the exponent is the right result
        h = sign | r;
    }
    return static_cast<int32_t>(static_cast<int16_t>(static_cast<uint16_t>(h)));
}
static int32_t bf16_bits(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x7FFFFFu)) return static_cast<int32_t>(static_cast<int16_t>(static_cast<uint16_t>((x >> 16) | 0x40u)));
    const uint32_t r = x + 0x7FFFu + ((x >> 16) & 1u);
    return static_cast<int32_t>(static_cast<int16_t>(static_cast<uint16_t>(r >> 16)));
}

nce_result_t ncePpeFuseClamp(nce_quant_t out, double clamp_min, double clamp_max, nce_ppe_task_t* ppe) {
    if (!ppe) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    if (out.dtype == NCE_DT_U8 || out.dtype == NCE_DT_I8) {
        if (out.scale == 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
        const double lo = std::round(clamp_min / out.scale) + out.zero_point;  // fuse_clamp.cpp:46-51
        const double hi = std::round(clamp_max / out.scale) + out.zero_point;
        // checked_cast<int32_t>: a value outside int32 is an error
        if (!(lo >= static_cast<double>(INT32_MIN) && lo <= static_cast<double>(INT32_MAX) && hi >= static_cast<double>(INT32_MIN) &&
              hi <= static_cast<double>(INT32_MAX)))
            return NCE_RESULT_ERROR_INVALID_ARGUMENT;
        ppe->clamp_low = std::max(ppe->clamp_low, static_cast<int32_t>(lo));
        ppe->clamp_high = std::min(ppe->clamp_high, static_cast<int32_t>(hi));
        return NCE_RESULT_SUCCESS;  // the mode stays (getPPEMode, :74-78)
    }
    if (out.dtype == NCE_DT_F16 || out.dtype == NCE_DT_BF16) {
        if (clamp_min != 0.0) return NCE_RESULT_ERROR_UNSUPPORTED;  // isLegalClamp: such a Clamp is not fused (:141-143)
        const int32_t bits = out.dtype == NCE_DT_F16 ? f16_bits(static_cast<float>(clamp_max)) : bf16_bits(static_cast<float>(clamp_max));
        ppe->clamp_low = INT32_MIN;
        ppe->clamp_high = std::min(ppe->clamp_high, bits);
        ppe->mode = NCE_PPE_LRELUX;  // :80-82
        return NCE_RESULT_SUCCESS;
    }
    return NCE_RESULT_ERROR_INVALID_ARGUMENT;
}

nce_result_t nceConvWeightSetBytes(int64_t ic, int64_t ky, int64_t kx, int64_t* set_bytes, int64_t* pad_bytes) {
    if (!set_bytes || !pad_bytes || ic <= 0 || ky <= 0 || kx <= 0 || ic > (1 << 24) || ky > 1024 || kx > 1024) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    const int64_t n = ic * ky * kx;  // 8-bit elements
    *set_bytes = (n + 15) / 16 * 16;
    *pad_bytes = *set_bytes - n;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceWeightsTableCheck(const int32_t* table, int32_t oc, int32_t weights_ptr_step) {
    if (!table || oc <= 0 || weights_ptr_step < 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    if (weights_ptr_step % 16 != 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;  // nce_sparsity.cpp:399-412
    const int64_t base = table[0];
    if (base % 16 != 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;             // :504-506
    for (int32_t c = 0; c < oc; ++c) {
        const int32_t* row = table + 4 * static_cast<int64_t>(c);
        if (static_cast<int64_t>(row[0]) - base != static_cast<int64_t>(c) * weights_ptr_step) return NCE_RESULT_ERROR_UNSUPPORTED;
        if (row[1] != 0xFFFFFF) return NCE_RESULT_ERROR_UNSUPPORTED;           // a sparsity map: not on this path
    }
    return NCE_RESULT_SUCCESS;
}

}  // extern "C"
