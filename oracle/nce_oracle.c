/*
 * nce_oracle.c - CPU ORACLE for the quantized NCE/DPU op path. TEST INFRASTRUCTURE ONLY
 * (see nce_oracle.h for what pins each function). Plain C, one file, OpenMP over output rows.
 *
 * Paths below are relative to the reference's src/vpux_compiler/src/ unless stated otherwise.
 */
#include "nce_oracle.h"

#include <limits.h>
#include <math.h>
#include <stddef.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ============================ parameter generation ========================================== */

/* utils/quantization.cpp:242-252. The mantissa is TRUNCATED toward zero by the double->integer
 * cast (checked_cast is a range check + static_cast). */
void nce_oracle_approximate(int bits, double target, int64_t* mult, int32_t* shift, int32_t* post_shift) {
    int exponent = 0;
    const double mantissa = frexp(target, &exponent);
    *mult = (int64_t)(mantissa * pow(2.0, bits));
    *shift = exponent > bits ? 0 : bits - exponent;
    *post_shift = exponent > bits ? bits - exponent : 0;
}

/* utils/quantization.cpp:256-264 */
int nce_oracle_quant_approx(int arch, double target, int32_t* mult, int32_t* shift, int32_t* post_shift) {
    int64_t m;
    int32_t s, ps;
    nce_oracle_approximate(15, target, &m, &s, &ps);
    if (m < 0 || m > 65535 || s < 0 || s > 255) return -1; /* checked_cast<uint16_t>/<uint8_t> */
    if (ps != 0 && arch != NCE_ORACLE_ARCH_30XX) return -1;
    *mult = (int32_t)m;
    *shift = s;
    *post_shift = ps;
    return 0;
}

/* utils/quantization.cpp:286-330 */
int nce_oracle_eltwise_approx(int arch, double in1_scale, double in2_scale, double out_scale, int32_t* in1_mult,
                              int32_t* in2_mult, int32_t* out_mult, int32_t* out_shift) {
    int32_t m1, s1, p1, m2, s2, p2, mo, so, po;
    if (nce_oracle_quant_approx(arch, in1_scale, &m1, &s1, &p1)) return -1;
    if (nce_oracle_quant_approx(arch, in2_scale, &m2, &s2, &p2)) return -1;
    if (nce_oracle_quant_approx(arch, 1.0 / out_scale, &mo, &so, &po)) return -1;
    const int64_t min_shift = s1 < s2 ? s1 : s2;
    const int64_t max_shift = s1 > s2 ? s1 : s2;
    const int64_t max_reg_shift = 63;
    const int64_t max_reg_mult = 65535;
    int to_max = 1;
    if (max_shift + so > max_reg_shift) to_max = 0;
    if (to_max && m1 > (max_reg_mult >> (max_shift - s1))) to_max = 0;
    if (to_max && m2 > (max_reg_mult >> (max_shift - s2))) to_max = 0;
    if (to_max) {
        m1 = (uint16_t)((int64_t)m1 << (max_shift - s1));
        m2 = (uint16_t)((int64_t)m2 << (max_shift - s2));
        so = (uint8_t)(so + max_shift);
    } else if (min_shift + so < max_reg_shift) {
        m1 = (uint16_t)((int64_t)m1 >> (s1 - min_shift));
        m2 = (uint16_t)((int64_t)m2 >> (s2 - min_shift));
        so = (uint8_t)(so + min_shift);
    } else {
        return -1;
    }
    *in1_mult = m1;
    *in2_mult = m2;
    *out_mult = mo;
    *out_shift = so;
    return 0;
}

/* utils/quantization.cpp:344-354 */
int nce_oracle_prelu_approx(int arch, double alpha, int32_t* mult, int32_t* shift) {
    const int bits = arch == NCE_ORACLE_ARCH_30XX ? 7 : 11;
    int64_t m;
    int32_t s, ps;
    nce_oracle_approximate(bits, alpha, &m, &s, &ps);
    if (ps != 0) return -1;
    *mult = (int32_t)m;
    *shift = s;
    return 0;
}

/* dialect/VPU/utils/nce_sparsity.cpp:122-155 (+ :227-232 for the 30XX LPRELU low byte) */
int32_t nce_oracle_scale_word(int arch, int32_t shift, int32_t mult, int32_t lrelu_mult) {
    uint32_t w;
    if (arch == NCE_ORACLE_ARCH_30XX) {
        w = (1u << 0) | ((uint32_t)shift << 8) | (1u << 14) | ((uint32_t)mult << 16);
        if (lrelu_mult >= 0) w = (w & 0xFFFFFF00u) | (uint32_t)lrelu_mult;
    } else {
        w = ((uint32_t)shift << 8) | ((uint32_t)mult << 16);
    }
    return (int32_t)w;
}

/* dialect/VPU/utils/nce_sparsity.cpp:31-33 */
int32_t nce_oracle_float_bits(double x) {
    const float f = (float)x;
    int32_t bits;
    memcpy(&bits, &f, sizeof(bits));
    return bits;
}

/* dialect/VPU/utils/nce_sparsity.cpp:186-193 and :646-676: bias / (w_scale * in_scale), refused
 * at or beyond the int32 limits, then std::round (half away from zero). */
int nce_oracle_rescaled_bias(double bias_fp, double w_scale, double in_scale, int32_t* out) {
    const double v = bias_fp / (w_scale * in_scale);
    if (v <= (double)INT32_MIN || v >= (double)INT32_MAX) return -1;
    *out = (int32_t)round(v);
    return 0;
}

/* dialect/VPU/utils/nce_sparsity.cpp:445-519 with getMultShiftFunc :224-283 (quantized in/out) */
int nce_oracle_weights_table(int arch, int32_t oc, int32_t weight_ptr_base, int32_t weight_ptr_step,
                             int32_t sparsity_ptr, double in_scale, double out_scale, const double* w_scales,
                             int32_t n_w_scales, const double* bias_fp, int32_t lrelu_mult, int32_t* table) {
    for (int32_t c = 0; c < oc; ++c) {
        const int32_t wptr = weight_ptr_base + c * weight_ptr_step;
        if (wptr % 16 != 0) return -1;
        if (sparsity_ptr != 0xFFFFFF && sparsity_ptr % 16 != 0) return -1;
        const double ws = n_w_scales == 1 ? w_scales[0] : w_scales[c];
        const double rescale = (ws * in_scale) / out_scale;
        int32_t m, s, ps;
        if (nce_oracle_quant_approx(arch, rescale, &m, &s, &ps)) return -1;
        int32_t b = 0;
        if (bias_fp != NULL && nce_oracle_rescaled_bias(bias_fp[c], ws, in_scale, &b)) return -1;
        table[4 * c + 0] = wptr;
        table[4 * c + 1] = sparsity_ptr; /* dense: same value for every channel (step 0) */
        table[4 * c + 2] = nce_oracle_scale_word(arch, s, m, lrelu_mult);
        table[4 * c + 3] = b;
    }
    return 0;
}

/* utils/VPU/ppe_utils.cpp:72-106 */
double nce_oracle_avgpool_scale(double in_scale, double out_scale, int32_t ky, int32_t kx) {
    return in_scale / out_scale / (double)((int64_t)ky * kx);
}

/* utils/VPU/ppe_utils.cpp:293-376; clamp for IE.Clamp: utils/quantization.cpp:364-380 */
int nce_oracle_ppe_stage1(int arch, int postop, double a0, double a1, int32_t storage_min, int32_t storage_max,
                          double out_scale, int32_t out_zp, nce_ppe_task_t* ppe) {
    const int64_t lo_q = (int64_t)storage_min - out_zp;
    const int64_t hi_q = (int64_t)storage_max - out_zp;
    ppe->lrelu_mult = 1;
    ppe->lrelu_shift = 0;
    ppe->clamp_domain = NCE_CLAMP_PRE_ZP;
    switch (postop) {
    case NCE_ORACLE_POSTOP_NONE: /* ppe_utils.cpp:151-156: storage range minus zero point */
        ppe->mode = NCE_PPE_NOOP;
        ppe->clamp_low = (int32_t)lo_q;
        ppe->clamp_high = (int32_t)hi_q;
        return 0;
    case NCE_ORACLE_POSTOP_RELU:
        ppe->mode = NCE_PPE_LRELU;
        ppe->clamp_low = 0;
        ppe->clamp_high = (int32_t)hi_q;
        return 0;
    case NCE_ORACLE_POSTOP_CLAMP: {
        const int64_t qmin = (int64_t)round(a0 / out_scale);
        const int64_t qmax = (int64_t)round(a1 / out_scale);
        ppe->mode = NCE_PPE_NOOP;
        ppe->clamp_low = (int32_t)(lo_q > qmin ? lo_q : qmin);
        ppe->clamp_high = (int32_t)(hi_q < qmax ? hi_q : qmax);
        return 0;
    }
    case NCE_ORACLE_POSTOP_LEAKY_RELU: {
        if (arch != NCE_ORACLE_ARCH_37XX) return -1; /* 30XX quantized LeakyReLU goes to the PWL table */
        ppe->mode = NCE_PPE_LPRELU;
        ppe->clamp_low = (int32_t)lo_q; /* slope is applied before clamping: no division by alpha */
        ppe->clamp_high = (int32_t)hi_q;
        const float af = (float)a0;
        if (fabsf(af - 0.0f) <= 1.1920929e-07f) { /* isFloatEqual(alpha, 0) */
            ppe->lrelu_mult = 0;
        } else if (!(fabsf(af - 1.0f) <= 1.1920929e-07f)) {
            if (nce_oracle_prelu_approx(arch, a0, &ppe->lrelu_mult, &ppe->lrelu_shift)) return -1;
        }
        return 0;
    }
    default:
        return -1;
    }
}

/* fuse_clamp.cpp:34-53: quantized bounds round(min / scale) + zp and round(max / scale) + zp (std::round: halves away
 * from zero), intersected with the range the op's PPE already has. */
int nce_oracle_fuse_clamp_quant(double out_scale, int32_t out_zp, double clamp_min, double clamp_max, int32_t* clamp_low,
                                int32_t* clamp_high) {
    if (out_scale == 0.0 || !clamp_low || !clamp_high) return -1;
    const double qlo = round(clamp_min / out_scale) + (double)out_zp;
    const double qhi = round(clamp_max / out_scale) + (double)out_zp;
    if (qlo < -2147483648.0 || qlo > 2147483647.0 || qhi < -2147483648.0 || qhi > 2147483647.0) return -1;
    if ((int32_t)qlo > *clamp_low) *clamp_low = (int32_t)qlo;
    if ((int32_t)qhi < *clamp_high) *clamp_high = (int32_t)qhi;
    return 0;
}

/* dialect/VPU/transforms/passes/setup_ppe.cpp:12-33 (mode) and :123-195 (clamps), quantized output */
void nce_oracle_ppe_stage2_37xx(int has_ppe, int32_t storage_min, int32_t storage_max, int32_t out_zp,
                                nce_ppe_task_t* ppe) {
    int32_t clamp_low = INT32_MIN, clamp_high = INT32_MAX, lrelu_mult = 1, lrelu_shift = 0;
    if (has_ppe) {
        clamp_low = ppe->clamp_low;
        clamp_high = ppe->clamp_high;
        lrelu_mult = ppe->lrelu_mult;
        lrelu_shift = ppe->lrelu_shift;
    }
    const int high_minus_zp = ((int64_t)storage_max - out_zp == clamp_high);
    int32_t mode;
    if (has_ppe && (lrelu_mult != 1 || lrelu_shift != 0)) {
        mode = NCE_PPE_LPRELU;
    } else if (high_minus_zp && clamp_low == 0) {
        mode = NCE_PPE_NOOP;
    } else if ((clamp_high == INT32_MAX || clamp_high == 0) && clamp_low == 0) {
        mode = NCE_PPE_LRELU;
    } else if (clamp_high < INT32_MAX && clamp_low == 0) {
        mode = NCE_PPE_LRELUX;
    } else {
        mode = NCE_PPE_NOOP;
    }
    int64_t new_low, new_high;
    if (mode == NCE_PPE_NOOP) {
        if (!has_ppe) {
            new_low = storage_min;
            new_high = storage_max;
        } else {
            new_low = (int64_t)clamp_low + out_zp;
            new_high = (int64_t)clamp_high + out_zp;
        }
    } else {
        new_low = storage_min;
        new_high = mode == NCE_PPE_LRELUX ? clamp_high : storage_max;
    }
    ppe->mode = mode;
    ppe->clamp_low = (int32_t)new_low;
    ppe->clamp_high = (int32_t)new_high;
    ppe->lrelu_mult = lrelu_mult;
    ppe->lrelu_shift = lrelu_shift;
    ppe->clamp_domain = NCE_CLAMP_POST_ZP;
}

/* ============================ per-element integer pipeline ================================== */

int64_t nce_oracle_rshift_round(int64_t p, int32_t s, int32_t round_mode) {
    if (s <= 0) return p;
    if (s > 63) s = 63;
    if (round_mode == NCE_ROUND_NONE) return p >> s;
    if (round_mode == NCE_ROUND_HALF_EVEN) {
        const int64_t q = p >> s;
        const int64_t r = p & (((int64_t)1 << s) - 1);
        const int64_t h = (int64_t)1 << (s - 1);
        return q + ((r > h) || (r == h && (q & 1)));
    }
    return (p + ((int64_t)1 << (s - 1))) >> s; /* HALF_UP */
}

static int64_t sat_i32(int64_t v) {
    return v > INT32_MAX ? INT32_MAX : (v < INT32_MIN ? INT32_MIN : v);
}

static void out_range(int32_t dtype, int64_t* lo, int64_t* hi) {
    if (dtype == NCE_DT_U8) {
        *lo = 0;
        *hi = 255;
    } else if (dtype == NCE_DT_I8) {
        *lo = -128;
        *hi = 127;
    } else {
        *lo = INT32_MIN;
        *hi = INT32_MAX;
    }
}

/* PReLU multiplier/shift from the mode: dialect/VPUMI37XX/ops/external/
 * runtime_dpu_parser_imports.cpp.inc:519-538 */
static void prelu_params(const nce_ppe_task_t* ppe, int64_t* pm, int32_t* ps) {
    *pm = 1;
    *ps = 0;
    if (ppe == NULL) return;
    if (ppe->mode == NCE_PPE_LPRELU) {
        *pm = ppe->lrelu_mult;
        *ps = ppe->lrelu_shift;
    } else if (ppe->mode == NCE_PPE_LRELU || ppe->mode == NCE_PPE_LRELUX) {
        *pm = 0;
        *ps = 0;
    }
}

int32_t nce_oracle_ppe(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const nce_ppe_task_t* ppe,
                       int32_t out_zp, int32_t out_dtype) {
    const int32_t rm = ppe ? ppe->round_mode : NCE_ROUND_HALF_UP;
    const int64_t clo = ppe ? ppe->clamp_low : INT32_MIN;
    const int64_t chi = ppe ? ppe->clamp_high : INT32_MAX;
    const int pre_zp = ppe ? ppe->clamp_domain == NCE_CLAMP_PRE_ZP : 0;
    int64_t pm;
    int32_t ps;
    prelu_params(ppe, &pm, &ps);

    int64_t x = (int64_t)acc + (int64_t)bias;                               /* 1 */
    x = sat_i32(nce_oracle_rshift_round(x * (int64_t)mult, shift, rm));     /* 2 */
    if (x < 0) x = sat_i32(nce_oracle_rshift_round(x * pm, ps, rm));        /* 3 */
    if (pre_zp) {
        x = x < clo ? clo : (x > chi ? chi : x);                            /* 5 */
        x += out_zp;                                                        /* 4 */
    } else {
        x += out_zp;                                                        /* 4 */
        x = x < clo ? clo : (x > chi ? chi : x);                            /* 5 */
    }
    int64_t lo, hi;
    out_range(out_dtype, &lo, &hi);
    x = x < lo ? lo : (x > hi ? hi : x);                                    /* 6 */
    return (int32_t)x;
}

static inline int32_t load8(const uint8_t* p, int32_t dtype) {
    return dtype == NCE_DT_I8 ? (int32_t)(int8_t)*p : (int32_t)*p;
}

static inline void store8(uint8_t* p, int32_t v) {
    *p = (uint8_t)(v & 0xFF);
}

/* Weights-table decode, 37XX integer packing: mult = bits 31:16, shift = bits 13:8
 * (dialect/VPU/utils/nce_sparsity.cpp:141-155; include/vpux/compiler/dialect/VPU37XX/
 * firmware_headers/details/api/vpu_nce_hw_37xx.h:240-249). */
static inline void table_decode(const int32_t* row, int32_t* mult, int32_t* shift, int32_t* bias) {
    const uint32_t w = (uint32_t)row[2];
    *mult = (int32_t)(w >> 16);
    *shift = (int32_t)((w >> 8) & 0x3F);
    *bias = row[3];
}

typedef struct {
    const nce_cluster_task_desc_t* t;
    int64_t N, C, H, W;     /* input */
    int64_t OC, OH, OW;     /* output */
    int KY, KX, SY, SX, PT, PL;
    int in_dt, w_dt, out_dt;
    int32_t zp_a, zp_w, zp_o;
    const uint8_t* in;
    const uint8_t* wt;
    const int32_t* table;
    uint8_t* out;
    int64_t is_n, is_h, is_w;   /* input strides (bytes) */
    int64_t ws_n, ws_h, ws_w;   /* weights / second-input strides */
    int64_t os_n, os_h, os_w, os_c;   /* output strides (os_c != 1: permuted output order) */
    int64_t tab_stride;         /* int32 elements between table rows */
} ctx_t;

static int32_t scale_for(const ctx_t* c, int64_t oc, int32_t* mult, int32_t* shift, int32_t* bias) {
    if (c->table != NULL) {
        table_decode(c->table + oc * c->tab_stride, mult, shift, bias);
        return 0;
    }
    const nce_ppe_task_t* p = c->t->ppe;
    if (p == NULL || !p->has_quant) return -1;
    *mult = p->quant_mult;
    *shift = p->quant_shift;
    *bias = 0;
    return 0;
}

/* One output element. Accumulation semantics: runtime_dpu_parser_imports.cpp.inc:834-945
 * (zero points removed before the MAC, padding contributes nothing), pools :1759-1905,
 * eltwise :1541-1555,1651-1757. The sum is kept in 64 bits and wrapped to int32 like a
 * 32-bit hardware accumulator. */
static void eval_element(const ctx_t* c, int64_t n, int64_t oy, int64_t ox, int64_t oc) {
    const nce_cluster_task_desc_t* t = c->t;
    uint8_t* dst = c->out + n * c->os_n + oy * c->os_h + ox * c->os_w + oc * c->os_c;
    int64_t acc = 0;
    switch (t->task_type) {
    case NCE_TASK_CONV: {
        const uint8_t* wrow = c->wt + oc * c->ws_n;
        for (int ky = 0; ky < c->KY; ++ky) {
            const int64_t iy = oy * c->SY + ky - c->PT;
            if (iy < 0 || iy >= c->H) continue;
            for (int kx = 0; kx < c->KX; ++kx) {
                const int64_t ix = ox * c->SX + kx - c->PL;
                if (ix < 0 || ix >= c->W) continue;
                const uint8_t* a = c->in + n * c->is_n + iy * c->is_h + ix * c->is_w;
                const uint8_t* w = wrow + ky * c->ws_h + kx * c->ws_w;
                int32_t s = 0;
                if (c->in_dt == NCE_DT_U8 && c->w_dt == NCE_DT_I8) { /* common case: let it vectorise */
                    for (int64_t ic = 0; ic < c->C; ++ic) s += ((int32_t)a[ic] - c->zp_a) * ((int32_t)(int8_t)w[ic] - c->zp_w);
                } else {
                    for (int64_t ic = 0; ic < c->C; ++ic)
                        s += (load8(a + ic, c->in_dt) - c->zp_a) * (load8(w + ic, c->w_dt) - c->zp_w);
                }
                acc += s;
            }
        }
        break;
    }
    case NCE_TASK_DWCONV: {
        const uint8_t* wrow = c->wt + oc * c->ws_n; /* one 16-byte-multiple row per channel, taps row-major */
        for (int ky = 0; ky < c->KY; ++ky) {
            const int64_t iy = oy * c->SY + ky - c->PT;
            if (iy < 0 || iy >= c->H) continue;
            for (int kx = 0; kx < c->KX; ++kx) {
                const int64_t ix = ox * c->SX + kx - c->PL;
                if (ix < 0 || ix >= c->W) continue;
                const int32_t a = load8(c->in + n * c->is_n + iy * c->is_h + ix * c->is_w + oc, c->in_dt);
                const int32_t w = load8(wrow + ky * c->KX + kx, c->w_dt);
                acc += (int64_t)(a - c->zp_a) * (w - c->zp_w);
            }
        }
        break;
    }
    case NCE_TASK_AVEPOOL: {
        for (int ky = 0; ky < c->KY; ++ky) {
            const int64_t iy = oy * c->SY + ky - c->PT;
            if (iy < 0 || iy >= c->H) continue;
            for (int kx = 0; kx < c->KX; ++kx) {
                const int64_t ix = ox * c->SX + kx - c->PL;
                if (ix < 0 || ix >= c->W) continue;
                acc += load8(c->in + n * c->is_n + iy * c->is_h + ix * c->is_w + oc, c->in_dt) - c->zp_a;
            }
        }
        break;
    }
    case NCE_TASK_MAXPOOL: {
        int64_t lo, hi;
        out_range(c->in_dt, &lo, &hi);
        int64_t m = lo;
        for (int ky = 0; ky < c->KY; ++ky) {
            const int64_t iy = oy * c->SY + ky - c->PT;
            if (iy < 0 || iy >= c->H) continue;
            for (int kx = 0; kx < c->KX; ++kx) {
                const int64_t ix = ox * c->SX + kx - c->PL;
                if (ix < 0 || ix >= c->W) continue;
                const int32_t a = load8(c->in + n * c->is_n + iy * c->is_h + ix * c->is_w + oc, c->in_dt);
                if (a > m) m = a;
            }
        }
        /* scale 1, shift 0, no rounding, output zero point forced to 0, clamp only
         * (runtime_dpu_parser_imports.cpp.inc:1790-1803, 2002-2004) */
        const int64_t clo = t->ppe ? t->ppe->clamp_low : INT32_MIN;
        const int64_t chi = t->ppe ? t->ppe->clamp_high : INT32_MAX;
        m = m < clo ? clo : (m > chi ? chi : m);
        out_range(c->out_dt, &lo, &hi);
        m = m < lo ? lo : (m > hi ? hi : m);
        store8(dst, (int32_t)m);
        return;
    }
    case NCE_TASK_ELTWISE: {
        const int32_t a = load8(c->in + n * c->is_n + oy * c->is_h + ox * c->is_w + oc, c->in_dt) - c->zp_a;
        const int32_t b = load8(c->wt + n * c->ws_n + oy * c->ws_h + ox * c->ws_w + oc, c->w_dt) - c->zp_w;
        if (t->ppe && t->ppe->has_in_mult)
            acc = (int64_t)t->ppe->in1_quant_mult * a + (int64_t)t->ppe->in2_quant_mult * b;
        else
            acc = (int64_t)a + b;
        break;
    }
    default:
        return;
    }
    int32_t mult = 1, shift = 0, bias = 0;
    scale_for(c, oc, &mult, &shift, &bias);
    const int32_t acc32 = (int32_t)(uint32_t)(uint64_t)acc;
    store8(dst, nce_oracle_ppe(acc32, bias, mult, shift, t->ppe, c->zp_o, c->out_dt));
}

int nce_oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

int nce_oracle_run(const nce_cluster_task_desc_t* t, int nthreads) {
    if (t == NULL || t->input.data == NULL || t->output.data == NULL || t->variants == NULL || t->num_variants == 0)
        return -1;
    ctx_t c;
    memset(&c, 0, sizeof(c));
    c.t = t;
    c.N = t->input.dims[0];
    c.C = t->input.dims[1];
    c.H = t->input.dims[2];
    c.W = t->input.dims[3];
    c.OC = t->output.dims[1];
    c.OH = t->output.dims[2];
    c.OW = t->output.dims[3];
    c.in_dt = t->input.dtype;
    c.w_dt = t->weights.dtype;
    c.out_dt = t->output.dtype;
    c.zp_a = t->input.zero_point;
    c.zp_w = t->weights.zero_point;
    c.zp_o = t->output.zero_point;
    c.in = (const uint8_t*)t->input.data;
    c.wt = (const uint8_t*)t->weights.data;
    c.out = (uint8_t*)t->output.data;
    c.is_n = t->input.strides_bytes[0];
    c.is_h = t->input.strides_bytes[2];
    c.is_w = t->input.strides_bytes[3];
    c.os_n = t->output.strides_bytes[0];
    c.os_h = t->output.strides_bytes[2];
    c.os_w = t->output.strides_bytes[3];
    c.os_c = t->output.strides_bytes[1];
    c.table = (const int32_t*)t->weight_table.data;
    c.tab_stride = c.table ? t->weight_table.strides_bytes[0] / 4 : 0;
    if (t->input.strides_bytes[1] != 1) return -2;
    if (t->output.dims[0] != c.N) return -2;

    switch (t->task_type) {
    case NCE_TASK_CONV:
        if (c.wt == NULL || c.table == NULL) return -3;
        if (t->weights.strides_bytes[1] != 1) return -2;
        c.ws_n = t->weights.strides_bytes[0];
        c.ws_h = t->weights.strides_bytes[2];
        c.ws_w = t->weights.strides_bytes[3];
        break;
    case NCE_TASK_DWCONV:
        if (c.wt == NULL || c.table == NULL) return -3;
        c.ws_n = t->weights.strides_bytes[0];
        break;
    case NCE_TASK_ELTWISE:
        if (c.wt == NULL) return -3;
        c.ws_n = t->weights.strides_bytes[0];
        c.ws_h = t->weights.strides_bytes[2];
        c.ws_w = t->weights.strides_bytes[3];
        if (c.table == NULL && !(t->ppe && t->ppe->has_quant)) return -4;
        break;
    case NCE_TASK_AVEPOOL:
        if (c.table == NULL && !(t->ppe && t->ppe->has_quant)) return -4;
        break;
    case NCE_TASK_MAXPOOL:
        break;
    default:
        return -5;
    }
    if (t->task_type == NCE_TASK_ELTWISE) {
        c.KY = c.KX = c.SY = c.SX = 1;
        c.PT = c.PL = 0;
    } else {
        c.KY = t->kernel_size[0];
        c.KX = t->kernel_size[1];
        c.SY = t->kernel_strides[0];
        c.SX = t->kernel_strides[1];
        c.PT = t->kernel_pad_top;
        c.PL = t->kernel_pad_left;
        if (c.KY < 1 || c.KX < 1 || c.SY < 1 || c.SX < 1) return -6;
    }
    for (uint32_t v = 0; v < t->num_variants; ++v) {
        const nce_dpu_task_t* d = &t->variants[v];
        if (d->out_start[0] < 0 || d->out_end[0] >= c.OW || d->out_start[1] < 0 || d->out_end[1] >= c.OH ||
            d->out_start[2] < 0 || d->out_end[2] >= c.OC)
            return -7;
    }
#ifdef _OPENMP
    const int nt = nthreads > 0 ? nthreads : omp_get_max_threads();
#else
    (void)nthreads;
#endif
    for (uint32_t v = 0; v < t->num_variants; ++v) {
        const nce_dpu_task_t* d = &t->variants[v];
        const int64_t rows = (int64_t)d->out_end[1] - d->out_start[1] + 1;
        if (rows <= 0) continue;
        const int64_t total = c.N * rows;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nt)
#endif
        for (int64_t r = 0; r < total; ++r) {
            const int64_t n = r / rows;
            const int64_t oy = d->out_start[1] + r % rows;
            for (int64_t ox = d->out_start[0]; ox <= d->out_end[0]; ++ox)
                for (int64_t oc = d->out_start[2]; oc <= d->out_end[2]; ++oc) eval_element(&c, n, oy, ox, oc);
        }
    }
    return 0;
}
