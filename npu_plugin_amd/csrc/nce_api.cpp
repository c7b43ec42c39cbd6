// Host side of the C-ABI declared in include/nce_hip.h: handles, log, descriptor validation
// (the rules of the reference's NCEClusterTaskOp verifier) and dispatch to the HIP kernels.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "nce_common.h"
#include "nce_conv_pk.h"
#include "nce_log.h"

struct nce_executor_s {
    int device = 0;
    nce_log_s* log = nullptr;
    nce::Options opt;  // tuning knobs, read from the environment once at creation
    // Persistent segments: a pinned host word their kernels raise when a bounded wait ran out (checked after a
    // synchronise; persistent launches are then switched off for this executor).
    uint32_t* pk_host_error = nullptr;
    std::atomic<bool> pk_off{false};
    // The library's fixed workspace on this executor's device (looked up at creation), for nceTaskListEnqueueNoAlloc.
    nce::PkWorkspace ws;
    bool ws_ok = false;
    std::atomic<bool> ws_used{false};   // a launch that reports through ws.error may be in flight
    // The workspace (error word, counters) is shared by every executor of the device: whichever executor reads a raised
    // error word clears it, so the failure is also counted per device (ws_failures below) and every executor compares
    // that count with the one it last saw.
    uint32_t ws_failures_seen = 0;
    // Pinned staging for the layer tables on their way into the workspace (made at creation, so that the enqueue itself
    // neither allocates nor leaves the runtime to pin pageable memory), and the event that says the last copy has left it.
    std::mutex ws_mu;
    uint8_t* ws_staging = nullptr;
    hipEvent_t ws_event = nullptr;
    bool ws_event_pending = false;
    ~nce_executor_s() {
        if (pk_host_error != nullptr) (void)hipHostFree(pk_host_error);
        if (ws_staging != nullptr) (void)hipHostFree(ws_staging);
        if (ws_event != nullptr) (void)hipEventDestroy(ws_event);
    }
};

thread_local nce::LaunchContext nce::tls_launch;

namespace {
// Launches of the fixed workspace that gave up, per device and process (see nce_executor_s::ws_failures_seen).
constexpr int kWsMaxDevices = 64;
std::atomic<uint32_t> ws_failures[kWsMaxDevices];
}  // namespace

namespace {

using nce::Box;
using nce::PpeDev;
using nce::TaskDev;
using nce::TensorDev;

constexpr int64_t kMaxKernel = 11;  // VPU::NCEInvariant::MAX_KERNEL_SIZE
constexpr int64_t kMaxStride = 8;   // NCE_MAX_STRIDE_SIZE, src/vpux_compiler/src/dialect/VPUIP/nce_invariant.cpp:1062

struct Plan {
    TaskDev dev;
    std::vector<Box> boxes;
    int task_type = 0;
};

// Sets the calling thread's launch context for the duration of one C-ABI call.
struct ScopedLaunch {
    nce::LaunchContext saved;
    ScopedLaunch(const nce::Options* opt, std::vector<nce::RecordedLaunch>* record, nce_log_s* log = nullptr) : saved(nce::tls_launch) {
        nce::tls_launch.opt = opt;
        nce::tls_launch.record = record;
        nce::tls_launch.log = log;
    }
    ~ScopedLaunch() { nce::tls_launch = saved; }
};

nce::Options read_options() {
    nce::Options o;
    if (const char* e = getenv("NCE_HIP_CONV_PATH")) {
        o.conv_path = atoi(e);
        o.env_path = true;
    }
    if (const char* e = getenv("NCE_HIP_CONV_WRES"))
        o.wres_forced = sscanf(e, "%d,%d,%d,%d", &o.wres[0], &o.wres[1], &o.wres[2], &o.wres[3]) == 4;
    if (const char* e = getenv("NCE_HIP_CONV_TILE")) o.halo_tile = atoi(e);
    if (const char* e = getenv("NCE_HIP_CONV_TILED")) o.tiled = atoi(e);
    if (const char* e = getenv("NCE_HIP_CONV_PATCH")) {
        int nf = 0, pr = 0, wv = 0, npx = 0;
        const int got = sscanf(e, "%d,%d,%d,%d", &nf, &pr, &wv, &npx);
        if (got >= 2) {
            o.patch = 1;
            o.patch_nf = nf;
            o.patch_pr = pr;
            o.patch_waves = got >= 3 ? wv : 0;
            o.patch_npx = got >= 4 ? npx : 0;
        } else if (got == 1) {
            o.patch = nf != 0 ? 1 : 0;
        }
    }
    o.no_fuse = getenv("NCE_HIP_NO_FUSE") != nullptr;
    if (const char* e = getenv("NCE_HIP_PERSISTENT")) o.persistent = atoi(e);
    if (const char* e = getenv("NCE_HIP_PERSISTENT_WAIT_US")) o.persistent_wait_us = std::max(0, atoi(e));
    return o;
}

#define FAIL(code, ...)              \
    do {                             \
        log->add(1, __VA_ARGS__);    \
        return code;                 \
    } while (0)

bool is_8bit(int32_t dt) {
    return dt == NCE_DT_U8 || dt == NCE_DT_I8;
}

void type_range(int32_t dt, int64_t* lo, int64_t* hi) {
    if (dt == NCE_DT_U8) {
        *lo = 0;
        *hi = 255;
    } else {
        *lo = -128;
        *hi = 127;
    }
}

int64_t clamp64(int64_t v, int64_t lo, int64_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

// Activation tensor: NHWC, channels compact and a multiple of 16 for 8-bit types
// (nce_cluster_task.cpp:346-359,702-709; src/vpux_compiler/src/dialect/VPU/utils/nce_invariant.cpp:135-153).
// An OUTPUT may instead be laid out in any order of H, W, C under N - the ODU permutations NWHC, NWCH, NCWH,
// NHCW, NCHW (getODUPermutationType, nce_cluster_task.cpp:764-780) - expressed through its strides: any
// non-overlapping strides are accepted and written byte by byte.
nce_result_t check_activation(nce_log_s* log, const char* name, const nce_tensor_t& x, TensorDev* out, bool allow_permuted = false) {
    if (x.data == nullptr) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: data pointer is null", name);
    if (!is_8bit(x.dtype)) FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "%s: only u8 / i8 storage is supported, got dtype %d", name, x.dtype);
    for (int i = 0; i < 4; ++i)
        if (x.dims[i] <= 0 || x.dims[i] > 0x7fffffff) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: dims[%d] = %lld", name, i, (long long)x.dims[i]);
    if (x.dims[1] % 16 != 0) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: channels (%lld) must be a multiple of 16", name, (long long)x.dims[1]);
    if (allow_permuted) {
        int order[4] = {0, 1, 2, 3};
        std::sort(order, order + 4, [&](int l, int r) { return x.strides_bytes[l] < x.strides_bytes[r]; });
        int64_t need = 1;
        for (int i = 0; i < 4; ++i) {
            const int d = order[i];
            if (x.dims[d] == 1) continue;  // the stride of an extent-1 dimension is never used
            if (x.strides_bytes[d] < need)
                FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: strides (N %lld, C %lld, H %lld, W %lld) make elements overlap", name,
                     (long long)x.strides_bytes[0], (long long)x.strides_bytes[1], (long long)x.strides_bytes[2], (long long)x.strides_bytes[3]);
            need = x.strides_bytes[d] * x.dims[d];
        }
        if (need > 0x7fffffff00LL) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: tensor too large", name);
        // compact channels are written with 128-bit stores
        if (x.strides_bytes[1] == 1 &&
            (((uintptr_t)x.data | (uintptr_t)x.strides_bytes[0] | (uintptr_t)x.strides_bytes[2] | (uintptr_t)x.strides_bytes[3]) & 15))
            FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "%s: data pointer and N/H/W strides must be 16-byte aligned", name);
    } else {
        if (x.strides_bytes[1] != 1) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: layout must be NHWC with compact channels (C stride %lld)", name, (long long)x.strides_bytes[1]);
        // ordered and non-overlapping: a pixel holds C bytes, a row W pixels, an image H rows (extent-1 dimensions aside);
        // the same size cap as for outputs
        const int64_t sw = x.strides_bytes[3], sh = x.strides_bytes[2], sn = x.strides_bytes[0];
        const bool ok_w = x.dims[3] == 1 || sw >= x.dims[1];
        const bool ok_h = x.dims[2] == 1 || (sh >= x.dims[1] && (x.dims[3] == 1 || sh / x.dims[3] >= sw));
        const bool ok_n = x.dims[0] == 1 || (sn >= x.dims[1] && (x.dims[3] == 1 || sn / x.dims[3] >= sw) && (x.dims[2] == 1 || sn / x.dims[2] >= sh));
        if (!ok_w || !ok_h || !ok_n)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: strides are not NHWC-ordered without overlap (N %lld, H %lld, W %lld, C 1)", name,
                 (long long)sn, (long long)sh, (long long)sw);
        int64_t span = x.dims[1];
        const int64_t ext[3] = {x.dims[3], x.dims[2], x.dims[0]}, str[3] = {sw, sh, sn};
        for (int i = 0; i < 3; ++i) {
            if (ext[i] > 1 && (str[i] > 0x7fffffff00LL / (ext[i] - 1))) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: tensor too large", name);
            span += (ext[i] - 1) * str[i];
        }
        if (span > 0x7fffffff00LL) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: tensor too large", name);
        if (((uintptr_t)x.data | (uintptr_t)x.strides_bytes[0] | (uintptr_t)x.strides_bytes[2] | (uintptr_t)x.strides_bytes[3]) & 15)
            FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "%s: data pointer and N/H/W strides must be 16-byte aligned", name);
    }
    int64_t lo, hi;
    type_range(x.dtype, &lo, &hi);
    if (x.zero_point < lo || x.zero_point > hi) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "%s: zero point %d outside the storage range", name, x.zero_point);
    out->data = static_cast<uint8_t*>(x.data);
    out->sn = x.strides_bytes[0];
    out->sh = x.strides_bytes[2];
    out->sw = x.strides_bytes[3];
    out->sc = x.strides_bytes[1];
    out->n = (int32_t)x.dims[0];
    out->c = (int32_t)x.dims[1];
    out->h = (int32_t)x.dims[2];
    out->w = (int32_t)x.dims[3];
    out->is_signed = x.dtype == NCE_DT_I8;
    out->zp = x.zero_point;
    return NCE_RESULT_SUCCESS;
}

// Weight table: [OC,1,1,4] si32, at least 4*OC elements (nce_cluster_task.cpp:361-416; shape
// src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:633-635).
nce_result_t check_table(nce_log_s* log, const nce_tensor_t& x, int64_t oc, TaskDev* dev) {
    if (x.dtype != NCE_DT_SI32) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weight_table: element type must be si32");
    int64_t elems = 1;
    for (int i = 0; i < 4; ++i) {
        if (x.dims[i] <= 0) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weight_table: dims[%d] = %lld", i, (long long)x.dims[i]);
        elems *= x.dims[i];
    }
    if (elems < 4 * oc) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weight_table: %lld elements, need %lld (4 per output channel)", (long long)elems, (long long)(4 * oc));
    if (x.strides_bytes[0] < 16 || x.strides_bytes[0] % 16 != 0 || ((uintptr_t)x.data & 15))
        FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weight_table: rows must be 16 bytes apart or more and 16-byte aligned");
    dev->table = static_cast<const int32_t*>(x.data);
    dev->table_stride = x.strides_bytes[0] / 4;
    return NCE_RESULT_SUCCESS;
}

// verifyKernel, src/vpux_compiler/src/dialect/VPUIP/nce_invariant.cpp:1056-1108 (37XX: SX may differ from SY).
nce_result_t check_kernel(nce_log_s* log, const nce_cluster_task_desc_t* t) {
    const int64_t KY = t->kernel_size[0], KX = t->kernel_size[1], SY = t->kernel_strides[0], SX = t->kernel_strides[1];
    if (KY <= 0 || KY > kMaxKernel) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "unsupported kernel height %lld, must be in [1, %lld]", (long long)KY, (long long)kMaxKernel);
    if (KX <= 0 || KX > kMaxKernel) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "unsupported kernel width %lld, must be in [1, %lld]", (long long)KX, (long long)kMaxKernel);
    if (SY <= 0 || SY > kMaxStride) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "unsupported stride height %lld, must be in [1, %lld]", (long long)SY, (long long)kMaxStride);
    if (SX <= 0 || SX > kMaxStride) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "unsupported stride width %lld, must be in [1, %lld]", (long long)SX, (long long)kMaxStride);
    const int64_t pads[4] = {t->kernel_pad_top, t->kernel_pad_bottom, t->kernel_pad_left, t->kernel_pad_right};
    const int64_t lim[4] = {KY / 2, KY / 2, KX / 2, KX / 2};
    for (int i = 0; i < 4; ++i)
        if (pads[i] < 0 || (pads[i] > 1 && pads[i] > lim[i]))
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "unsupported padding %lld, must be in [0, %lld]", (long long)pads[i], (long long)std::max<int64_t>(1, lim[i]));
    return NCE_RESULT_SUCCESS;
}

nce_result_t check_out_shape(nce_log_s* log, const nce_cluster_task_desc_t* t, const TensorDev& in, const TensorDev& out) {
    const int64_t eh = ((int64_t)in.h + t->kernel_pad_top + t->kernel_pad_bottom - t->kernel_size[0]) / t->kernel_strides[0] + 1;
    const int64_t ew = ((int64_t)in.w + t->kernel_pad_left + t->kernel_pad_right - t->kernel_size[1]) / t->kernel_strides[1] + 1;
    if ((int64_t)in.h + t->kernel_pad_top + t->kernel_pad_bottom < t->kernel_size[0] ||
        (int64_t)in.w + t->kernel_pad_left + t->kernel_pad_right < t->kernel_size[1])
        FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "kernel is larger than the padded input");
    if (out.h != eh || out.w != ew)
        FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "output is %dx%d, kernel/stride/pad give %lldx%lld", out.h, out.w, (long long)eh, (long long)ew);
    if (out.n != in.n) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "output batch %d differs from input batch %d", out.n, in.n);
    return NCE_RESULT_SUCCESS;
}

// PPETask -> the form the kernels use. Mode handling follows setupQuantInQuantOut
// (runtime_dpu_parser_imports.cpp.inc:511-542); limits of the PReLU registers:
// src/vpux_compiler/src/dialect/VPU/transforms/passes/setup_ppe.cpp:77-92.
nce_result_t build_ppe(nce_log_s* log, const nce_cluster_task_desc_t* t, const nce_tensor_t& out, bool has_table, PpeDev* d) {
    static const nce_ppe_task_t kDefault = {NCE_PPE_NOOP, INT32_MIN, INT32_MAX, 1, 0, 0, 1, 0, 0, 0, 1, 1, NCE_ROUND_HALF_UP, NCE_CLAMP_POST_ZP};
    const nce_ppe_task_t& p = t->ppe ? *t->ppe : kDefault;
    d->prelu_mult = 1;
    d->prelu_shift = 0;
    switch (p.mode) {
    case NCE_PPE_NOOP:
    case NCE_PPE_ADD:
        break;
    case NCE_PPE_LRELU:
    case NCE_PPE_LRELUX:
        d->prelu_mult = 0;
        break;
    case NCE_PPE_LPRELU: {
        const int64_t am = p.lrelu_mult < 0 ? -(int64_t)p.lrelu_mult : p.lrelu_mult;
        if (am & ~(int64_t)0x7FF) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: ReLU multiplier %d exceeds 11 bits", p.lrelu_mult);
        if (p.lrelu_shift & ~0x1F) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: ReLU shift %d does not fit 5 bits", p.lrelu_shift);
        d->prelu_mult = p.lrelu_mult;
        d->prelu_shift = p.lrelu_shift;
        break;
    }
    default:
        FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "ppe: mode %d is not part of the INT8 path", p.mode);
    }
    if (p.round_mode < NCE_ROUND_HALF_UP || p.round_mode > NCE_ROUND_NONE) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: round_mode %d", p.round_mode);
    if (p.clamp_domain != NCE_CLAMP_POST_ZP && p.clamp_domain != NCE_CLAMP_PRE_ZP) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: clamp_domain %d", p.clamp_domain);
    if (p.clamp_low > p.clamp_high) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: clamp_low %d > clamp_high %d", p.clamp_low, p.clamp_high);
    d->round_mode = p.round_mode;

    int64_t tlo, thi;
    type_range(out.dtype, &tlo, &thi);
    const bool is_max = t->task_type == NCE_TASK_MAXPOOL;
    const int64_t zp = is_max ? 0 : out.zero_point;  // MAXPOOL: zero point register forced to 0 (…inc:2002-2004)
    int64_t lo = p.clamp_low, hi = p.clamp_high;
    if (p.clamp_domain == NCE_CLAMP_PRE_ZP && !is_max) {
        lo += zp;
        hi += zp;
    }
    d->lo = (int32_t)(clamp64(lo, tlo, thi) - zp);
    d->hi = (int32_t)(clamp64(hi, tlo, thi) - zp);
    d->zp_out = (int32_t)zp;
    if (!is_max && d->prelu_mult == 0) {
        // slope 0 (ReLU): negative values become 0 before the clamp, which is the clamp with its
        // lower bound raised to 0 - the kernels then skip the PReLU step altogether
        d->prelu_mult = 1;
        d->prelu_shift = 0;
        if (d->lo < 0) d->lo = 0;
        if (d->hi < d->lo) d->lo = d->hi;
    }

    d->quant_mult = 1;
    d->quant_shift = 0;
    d->in1_mult = d->in2_mult = 1;
    const bool needs_quant = (t->task_type == NCE_TASK_ELTWISE || t->task_type == NCE_TASK_AVEPOOL) && !has_table;
    if (needs_quant) {
        if (!p.has_quant) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: task has no weight table, so quant_mult / quant_shift are required");
        if (p.quant_mult < 0 || p.quant_mult > 65535) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: quant_mult %d does not fit 16 bits", p.quant_mult);
        if (p.quant_shift < 0 || p.quant_shift > 63) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: quant_shift %d does not fit 6 bits", p.quant_shift);
        if (p.quant_post_shift != 0) FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "ppe: quant_post_shift is a 30XX feature");
        d->quant_mult = p.quant_mult;
        d->quant_shift = p.quant_shift;
    }
    if (t->task_type == NCE_TASK_ELTWISE && p.has_in_mult) {
        if (p.in1_quant_mult < 0 || p.in1_quant_mult > 65535 || p.in2_quant_mult < 0 || p.in2_quant_mult > 65535)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ppe: in1/in2_quant_mult must fit 16 bits");
        d->in1_mult = p.in1_quant_mult;
        d->in2_mult = p.in2_quant_mult;
    }
    return NCE_RESULT_SUCCESS;
}

int64_t box_volume(const Box& b) {
    return (int64_t)b.bw * b.bh * b.bc;
}

bool boxes_overlap(const Box& a, const Box& b) {
    return a.x0 < b.x0 + b.bw && b.x0 < a.x0 + a.bw && a.y0 < b.y0 + b.bh && b.y0 < a.y0 + a.bh && a.z0 < b.z0 + b.bc &&
           b.z0 < a.z0 + a.bc;
}

// DPUTask variants: 3-D inclusive boxes inside the output (nce_cluster_task.cpp:588-608,643-663).
nce_result_t build_boxes(nce_log_s* log, const nce_cluster_task_desc_t* t, const TensorDev& in, const TensorDev& out, std::vector<Box>* boxes) {
    if (t->variants == nullptr || t->num_variants == 0) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "task must have at least one DPUTask variant");
    boxes->clear();
    for (uint32_t v = 0; v < t->num_variants; ++v) {
        const nce_dpu_task_t& d = t->variants[v];
        const int32_t dim[3] = {out.w, out.h, out.c};
        for (int i = 0; i < 3; ++i)
            if (d.out_start[i] < 0 || d.out_end[i] < d.out_start[i] || d.out_end[i] >= dim[i])
                FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "variant %u: out_start/out_end[%d] = %d..%d outside 0..%d", v, i, d.out_start[i], d.out_end[i], dim[i] - 1);
        if (d.out_start[2] % 16 != 0 || (d.out_end[2] + 1) % 16 != 0)
            FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "variant %u: channel range %d..%d must cover whole groups of 16", v, d.out_start[2], d.out_end[2]);
        if (d.mpe_mode < NCE_MPE_VECTOR || d.mpe_mode > NCE_MPE_NOP) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "variant %u: mpe_mode %d", v, d.mpe_mode);
        if (t->task_type != NCE_TASK_ELTWISE) {
            // The pad a variant carries is the part of the kernel padding its box touches; the GPU
            // kernels derive it from global coordinates, so a different value is only reported.
            const int64_t last_y = (int64_t)d.out_end[1] * t->kernel_strides[0] - t->kernel_pad_top + t->kernel_size[0] - 1;
            const int64_t last_x = (int64_t)d.out_end[0] * t->kernel_strides[1] - t->kernel_pad_left + t->kernel_size[1] - 1;
            const int64_t et = std::max<int64_t>(0, t->kernel_pad_top - (int64_t)d.out_start[1] * t->kernel_strides[0]);
            const int64_t el = std::max<int64_t>(0, t->kernel_pad_left - (int64_t)d.out_start[0] * t->kernel_strides[1]);
            const int64_t eb = std::max<int64_t>(0, last_y - (in.h - 1));
            const int64_t er = std::max<int64_t>(0, last_x - (in.w - 1));
            if (d.pad_top != et || d.pad_bottom != eb || d.pad_left != el || d.pad_right != er)
                log->add(2, "variant %u: pad {l %d, r %d, t %d, b %d} differs from the geometry {l %lld, r %lld, t %lld, b %lld}; geometry is used",
                         v, d.pad_left, d.pad_right, d.pad_top, d.pad_bottom, (long long)el, (long long)er, (long long)et, (long long)eb);
        }
        Box b;
        b.x0 = d.out_start[0];
        b.y0 = d.out_start[1];
        b.z0 = d.out_start[2];
        b.bw = d.out_end[0] - d.out_start[0] + 1;
        b.bh = d.out_end[1] - d.out_start[1] + 1;
        b.bc = d.out_end[2] - d.out_start[2] + 1;
        boxes->push_back(b);
    }
    // Variants that tile the whole output exactly are one launch over the full box: every output
    // element is a pure function of its coordinates, so the bytes are the same for any tiling.
    if (boxes->size() > 1 && boxes->size() <= 1024) {
        int64_t vol = 0;
        for (const Box& b : *boxes) vol += box_volume(b);
        bool exact = vol == (int64_t)out.w * out.h * out.c;
        for (size_t i = 0; exact && i < boxes->size(); ++i)
            for (size_t j = i + 1; exact && j < boxes->size(); ++j)
                if (boxes_overlap((*boxes)[i], (*boxes)[j])) exact = false;
        if (exact) {
            Box full = {0, 0, 0, out.w, out.h, out.c};
            boxes->assign(1, full);
        }
    }
    return NCE_RESULT_SUCCESS;
}

nce_result_t make_plan(nce_log_s* log, const nce_cluster_task_desc_t* t, Plan* plan) {
    if (t == nullptr) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "task descriptor is null");
    // is_inplace is the one boolean attribute with a meaning here (below, with the ELTWISE checks); the others change what the
    // hardware computes or how operands are stored.
    if ((t->flags & ~NCE_FLAG_IS_INPLACE) != 0)
        FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "task flags 0x%x: continued / segmented / compressed / superdense / permute-quantize / small-kernel tasks are not supported", t->flags & ~NCE_FLAG_IS_INPLACE);
    if ((t->flags & NCE_FLAG_IS_INPLACE) != 0 && t->task_type != NCE_TASK_ELTWISE)
        FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "is_inplace is an attribute of ELTWISE tasks");
    TaskDev& d = plan->dev;
    memset(&d, 0, sizeof(d));
    plan->task_type = t->task_type;
    switch (t->task_type) {
    case NCE_TASK_CONV:
    case NCE_TASK_DWCONV:
    case NCE_TASK_MAXPOOL:
    case NCE_TASK_AVEPOOL:
    case NCE_TASK_ELTWISE:
        break;
    default:
        FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "task_type %d is not supported (CONV, DWCONV, MAXPOOL, AVEPOOL, ELTWISE are)", t->task_type);
    }
    nce_result_t r;
    if ((r = check_activation(log, "input", t->input, &d.in)) != NCE_RESULT_SUCCESS) return r;
    if ((r = check_activation(log, "output", t->output, &d.out, true)) != NCE_RESULT_SUCCESS) return r;

    const bool has_table = t->weight_table.data != nullptr;
    if (has_table && (r = check_table(log, t->weight_table, d.out.c, &d)) != NCE_RESULT_SUCCESS) return r;

    if (t->task_type == NCE_TASK_ELTWISE) {
        // nce_cluster_task.cpp:522-584: no kernel attributes, second input required, same shapes.
        if (t->kernel_size[0] > 1 || t->kernel_size[1] > 1 || t->kernel_strides[0] > 1 || t->kernel_strides[1] > 1)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ELTWISE must not carry kernel_size / kernel_strides");
        if (t->kernel_pad_left || t->kernel_pad_right || t->kernel_pad_top || t->kernel_pad_bottom)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ELTWISE must not carry padding");
        if ((r = check_activation(log, "weights (second eltwise input)", t->weights, &d.in2)) != NCE_RESULT_SUCCESS) return r;
        if (d.in2.n != d.in.n || d.in2.c != d.in.c || d.in2.h != d.in.h || d.in2.w != d.in.w || d.out.n != d.in.n ||
            d.out.c != d.in.c || d.out.h != d.in.h || d.out.w != d.in.w)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ELTWISE inputs and output must have the same shape (no broadcast)");
        if (d.in2.is_signed != d.in.is_signed)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "ELTWISE inputs must share the storage type");  // eltwise_utils.cpp:15-65
        d.ky = d.kx = d.sy = d.sx = 1;
        if ((t->flags & NCE_FLAG_IS_INPLACE) != 0) {
            // The reference replaces an in-place eltwise's output buffer by one of its input buffers, which must have the
            // output's element type and allocation size (convert_eltwise_to_in_place.cpp:114-200): the output must BE one of
            // the inputs. Every output element depends on the same element of the inputs only, so the kernels need nothing else.
            const auto same = [](const nce::TensorDev& x, const nce::TensorDev& y) {
                return x.data == y.data && x.sn == y.sn && x.sh == y.sh && x.sw == y.sw && x.sc == y.sc && x.is_signed == y.is_signed;
            };
            if (!same(d.out, d.in) && !same(d.out, d.in2))
                FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "is_inplace: the output must be one of the two inputs (same address, strides and storage type)");
        }
    } else {
        if ((r = check_kernel(log, t)) != NCE_RESULT_SUCCESS) return r;
        if ((r = check_out_shape(log, t, d.in, d.out)) != NCE_RESULT_SUCCESS) return r;
        d.ky = t->kernel_size[0];
        d.kx = t->kernel_size[1];
        d.sy = t->kernel_strides[0];
        d.sx = t->kernel_strides[1];
        d.pt = t->kernel_pad_top;
        d.pl = t->kernel_pad_left;
        d.pr = t->kernel_pad_right;
    }

    const nce_tensor_t& w = t->weights;
    if (t->task_type == NCE_TASK_CONV || t->task_type == NCE_TASK_DWCONV) {
        if (w.data == nullptr) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weights are required");          // nce_cluster_task.cpp:361-378
        if (!has_table) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weight_table is required");             // nce_cluster_task.cpp:379-398
        if (!is_8bit(w.dtype)) FAIL(NCE_RESULT_ERROR_UNSUPPORTED, "weights: only u8 / i8 storage is supported");
        int64_t lo, hi;
        type_range(w.dtype, &lo, &hi);
        if (w.zero_point < lo || w.zero_point > hi) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weights: zero point %d outside the storage range", w.zero_point);
        if (((uintptr_t)w.data | (uintptr_t)w.strides_bytes[0]) & 15)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weights: every weight set must start on a 16-byte boundary");  // nce_sparsity.cpp:504-506
        d.weights = static_cast<const uint8_t*>(w.data);
        d.w_stride_oc = w.strides_bytes[0];
        d.w_is_signed = w.dtype == NCE_DT_I8;
        d.w_zp = w.zero_point;
    }
    if (t->task_type == NCE_TASK_CONV) {
        // OYXI: [OC, IC, KY, KX] logical, IC innermost in memory (nce_cluster_task.cpp:418-433).
        if (w.dims[0] != d.out.c || w.dims[1] != d.in.c || w.dims[2] != d.ky || w.dims[3] != d.kx)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weights dims [%lld,%lld,%lld,%lld] do not match [OC %d, IC %d, KY %d, KX %d]",
                 (long long)w.dims[0], (long long)w.dims[1], (long long)w.dims[2], (long long)w.dims[3], d.out.c, d.in.c, d.ky, d.kx);
        if (w.strides_bytes[1] != 1 || w.strides_bytes[3] != d.in.c || w.strides_bytes[2] != (int64_t)d.kx * d.in.c ||
            w.strides_bytes[0] < (int64_t)d.ky * d.kx * d.in.c)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "weights must be OYXI with compact weight sets");
    } else if (t->task_type == NCE_TASK_DWCONV) {
        // [C, pad16(KY*KX), 1, 1]: one row per channel (const_utils.cpp:216-243; nce_depth_convolution.cpp:93-108).
        if (d.out.c != d.in.c) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "DWCONV: output channels %d must equal input channels %d", d.out.c, d.in.c);
        if (w.dims[0] != d.in.c || w.dims[1] < (int64_t)d.ky * d.kx || w.dims[1] % 16 != 0 || w.dims[2] != 1 || w.dims[3] != 1)
            FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "DWCONV weights must be [C, pad16(KY*KX), 1, 1], got [%lld,%lld,%lld,%lld]",
                 (long long)w.dims[0], (long long)w.dims[1], (long long)w.dims[2], (long long)w.dims[3]);
        if (w.strides_bytes[1] != 1 || w.strides_bytes[0] < w.dims[1]) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "DWCONV weight rows must be compact");
    } else if (t->task_type == NCE_TASK_MAXPOOL || t->task_type == NCE_TASK_AVEPOOL) {
        if (d.out.c != d.in.c) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "pooling: output channels %d must equal input channels %d", d.out.c, d.in.c);
        if (t->task_type == NCE_TASK_MAXPOOL) {
            if (t->output.dtype != t->input.dtype) FAIL(NCE_RESULT_ERROR_INVALID_ARGUMENT, "MAXPOOL: input and output storage types must match");
            d.table = nullptr;  // no scale, no bias on this path
        }
    }

    if ((r = build_ppe(log, t, t->output, d.table != nullptr, &d.ppe)) != NCE_RESULT_SUCCESS) return r;
    return build_boxes(log, t, d.in, d.out, &plan->boxes);
}

nce_result_t launch_plan(nce_executor_s* ex, const Plan& plan, hipStream_t stream) {
    for (const Box& b : plan.boxes) {
        hipError_t e = hipSuccess;
        switch (plan.task_type) {
        case NCE_TASK_CONV: e = nce::launch_conv(plan.dev, b, stream); break;
        case NCE_TASK_DWCONV: e = nce::launch_dwconv(plan.dev, b, stream); break;
        case NCE_TASK_MAXPOOL: e = nce::launch_pool(plan.dev, b, true, stream); break;
        case NCE_TASK_AVEPOOL: e = nce::launch_pool(plan.dev, b, false, stream); break;
        case NCE_TASK_ELTWISE: e = nce::launch_eltwise(plan.dev, b, stream); break;
        }
        if (e != hipSuccess) {
            ex->log->add(1, "kernel launch failed: %s", hipGetErrorString(e));
            return NCE_RESULT_ERROR_UNKNOWN;
        }
    }
    return NCE_RESULT_SUCCESS;
}

}  // namespace

// A task list keeps the validated plans and, from its first Enqueue on, the prepared launches (kernel, grid and
// argument block of every launch, conv + add pairs already fused): an Enqueue is then a loop of hipLaunchKernel.
struct nce_task_list_s {
    nce_executor_s* ex = nullptr;
    std::mutex mu;
    std::vector<Plan> plans;
    std::vector<nce::RecordedLaunch> launches;
    std::vector<void*> device_mem;  // tables and counters of persistent segments (none in the fixed-workspace form)
    std::vector<uint8_t> ws_table;  // fixed-workspace form: the segments' tables, copied to the workspace by every enqueue
    bool prepared = false;
    bool fixed_ws = false;          // prepared for the fixed workspace
    bool has_segments = false;
    void drop_prepared() {
        for (void* p : device_mem) (void)hipFree(p);
        device_mem.clear();
        ws_table.clear();
        launches.clear();
        prepared = false;
        fixed_ws = false;
        has_segments = false;
    }
    ~nce_task_list_s() { drop_prepared(); }
};

namespace {

// ---- persistent segments (nce_conv_pk.h) -----------------------------------------------------------------------------------
// A tensor a layer touches, for the question whether a run of layers may share one persistent launch: every XCD works on
// its own eighth of the batch and runs ahead of or behind the others, so two layers of a segment may touch the same memory
// only if both cut it into the same eight shares (same base, batch and batch stride) - or if both only read it.
struct PkTensor {
    const uint8_t* lo;
    const uint8_t* hi;
    int64_t sn;
    int32_t n;        // 0: not cut by batch (weights, tables)
    bool written;
};
PkTensor pk_tensor(const nce::TensorDev& t, bool written) {
    return {t.data, t.data + (int64_t)t.n * t.sn, t.sn, t.n, written};
}
bool pk_conflict(const PkTensor& x, const PkTensor& y) {
    if (!(x.lo < y.hi && y.lo < x.hi)) return false;
    if (!x.written && !y.written) return false;
    return !(x.n != 0 && x.lo == y.lo && x.n == y.n && x.sn == y.sn);
}

// The per-XCD form of one recorded launch (a convolution, possibly with its fused residual add), if it has one.
struct PkAlt {
    bool ok = false;
    nce::RecordedLaunch launch;          // recorded with an eighth of the batch for 32 CUs
    int64_t d_in = 0, d_out = 0, d_other = 0, d_fzout = 0;
    std::vector<PkTensor> tensors;
};

PkAlt pk_alternate(const Plan& p, const Plan* q) {
    PkAlt alt;
    const int32_t n = p.dev.out.n;
    if (p.boxes.size() != 1 || n % 8 != 0 || p.dev.in.n != n) return alt;
    if (q != nullptr && (q->boxes.size() != 1 || q->dev.in.n != n || q->dev.in2.n != n || q->dev.out.n != n)) return alt;
    TaskDev pd = p.dev;
    pd.in.n = pd.out.n = n / 8;
    std::vector<nce::RecordedLaunch> rec;
    hipError_t e;
    {
        const ScopedLaunch ctx(nce::tls_launch.opt, &rec);  // (restores the caller's recorder, also when a launch throws)
        nce::tls_launch.per_xcd = true;
        if (q != nullptr) {
            TaskDev qd = q->dev;
            qd.in.n = qd.in2.n = qd.out.n = n / 8;
            e = nce::launch_conv_fused_add(pd, p.boxes[0], qd, q->boxes[0], nullptr);
        } else {
            e = nce::launch_conv(pd, p.boxes[0], nullptr);
        }
    }
    if (e != hipSuccess || rec.size() != 1 || !nce::wres_pk_has_variant(rec[0].tag)) return alt;
    alt.launch = std::move(rec[0]);
    alt.d_in = (int64_t)(n / 8) * p.dev.in.sn;
    alt.d_out = (int64_t)(n / 8) * p.dev.out.sn;
    alt.tensors.push_back(pk_tensor(p.dev.in, false));
    alt.tensors.push_back(pk_tensor(p.dev.out, true));
    alt.tensors.push_back({p.dev.weights, p.dev.weights + (int64_t)p.dev.out.c * p.dev.w_stride_oc, 0, 0, false});
    const uint8_t* const tb = reinterpret_cast<const uint8_t*>(p.dev.table);
    alt.tensors.push_back({tb, tb + (int64_t)p.dev.out.c * p.dev.table_stride * 4, 0, 0, false});
    if (q != nullptr) {
        const nce::TensorDev& other = q->dev.in.data == p.dev.out.data ? q->dev.in2 : q->dev.in;
        alt.d_other = (int64_t)(n / 8) * other.sn;
        alt.d_fzout = (int64_t)(n / 8) * q->dev.out.sn;
        alt.tensors.push_back(pk_tensor(other, false));
        alt.tensors.push_back(pk_tensor(q->dev.out, true));
    }
    alt.ok = true;
    return alt;
}

// Walk the plans the way they are to run (stream order), launching or - with a recorder set - recording. alts (recording
// only, optional) receives one entry per recorded launch: its per-XCD form where it has one.
nce_result_t run_plans(nce_executor_s* ex, const std::vector<Plan>& plans, hipStream_t stream, std::vector<PkAlt>* alts = nullptr) {
    const auto note = [&](PkAlt&& alt) {
        if (alts == nullptr) return;
        while (alts->size() + 1 < nce::tls_launch.record->size()) alts->emplace_back();  // launches without an alternate
        alts->push_back(std::move(alt));
    };
    for (size_t i = 0; i < plans.size(); ++i) {
        const Plan& p = plans[i];
        // A convolution directly followed by the residual add that consumes its output runs as one launch where the
        // kernels allow it (both outputs are written; the bytes are those of the two tasks run one after the other).
        if (p.task_type == NCE_TASK_CONV && p.boxes.size() == 1 && i + 1 < plans.size()) {
            const Plan& q = plans[i + 1];
            if (q.task_type == NCE_TASK_ELTWISE && q.boxes.size() == 1) {
                const hipError_t e = nce::launch_conv_fused_add(p.dev, p.boxes[0], q.dev, q.boxes[0], stream);
                if (e == hipSuccess) {
                    if (alts != nullptr) note(pk_alternate(p, &q));
                    ++i;
                    continue;
                }
                if (e != hipErrorNotSupported) {
                    ex->log->add(1, "kernel launch failed: %s", hipGetErrorString(e));
                    return NCE_RESULT_ERROR_UNKNOWN;
                }
            }
        }
        const nce_result_t r = launch_plan(ex, p, stream);
        if (r != NCE_RESULT_SUCCESS) return r;
        if (alts != nullptr && p.task_type == NCE_TASK_CONV && p.boxes.size() == 1) note(pk_alternate(p, nullptr));
    }
    if (alts != nullptr) alts->resize(nce::tls_launch.record->size());
    return NCE_RESULT_SUCCESS;
}

// Replace every run of two or more consecutive launches that have a per-XCD form (and whose tensors allow it) by one
// persistent launch. Allocates the segments' device tables and counters (kept in list->device_mem) - or, with fixed_ws,
// allocates nothing: the tables are gathered in list->ws_table for the executor's fixed workspace, whose counters and error
// word the launches use.
nce_result_t build_segments(nce_task_list_s* list, std::vector<PkAlt>& alts, bool fixed_ws) {
    nce_executor_s* const ex = list->ex;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ex->device) != hipSuccess || cus != nce::kPkWorkgroups) return NCE_RESULT_SUCCESS;
    if (!fixed_ws && ex->pk_host_error == nullptr) return NCE_RESULT_SUCCESS;  // (no error word: no persistent launches)
    std::vector<nce::RecordedLaunch> out;
    size_t i = 0;
    const size_t n = list->launches.size();
    while (i < n) {
        // the longest run from i whose tensors do not conflict
        size_t j = i;
        std::vector<PkTensor> seen;
        while (j < n && alts[j].ok && j - i < (size_t)nce::kPkMaxLayers) {
            bool clash = false;
            for (const PkTensor& t : alts[j].tensors)
                for (const PkTensor& u : seen) clash = clash || pk_conflict(t, u);
            if (clash) break;
            seen.insert(seen.end(), alts[j].tensors.begin(), alts[j].tensors.end());
            ++j;
        }
        if (j - i < 2) {
            out.push_back(std::move(list->launches[i]));
            ++i;
            continue;
        }
        std::vector<nce::PkLayerDesc> layers;
        for (size_t k = i; k < j; ++k) layers.push_back({&alts[k].launch, alts[k].d_in, alts[k].d_out, alts[k].d_other, alts[k].d_fzout});
        std::vector<uint8_t> table;
        nce::RecordedLaunch seg;
        const hipError_t e = nce::wres_pk_make(layers, &table, &seg);
        void* d_table = nullptr;
        void* d_ctl = nullptr;
        if (fixed_ws && e == hipSuccess) {
            if (list->ws_table.size() + table.size() > ex->ws.table_bytes) {
                // The workspace holds the tables of kPkMaxLayers layers per list: what does not fit runs as the ordinary
                // recorded launches it was made from (which allocate nothing either).
                ex->log->add(2, "task list: launches %zu..%zu stay ordinary launches (the fixed workspace holds %d layers per list)",
                             i, j - 1, nce::kPkMaxLayers);
                for (size_t k = i; k < j; ++k) out.push_back(std::move(list->launches[k]));
                i = j;
                continue;
            }
            nce::PkArgs args;
            args.layers = ex->ws.table + list->ws_table.size();
            args.ctl = ex->ws.ctl;
            args.host_error = ex->ws.error;
            args.nlayers = (int32_t)(j - i);
            args.wait_us = (uint32_t)ex->opt.persistent_wait_us;
            list->ws_table.insert(list->ws_table.end(), table.begin(), table.end());
            seg.arg.resize((sizeof(args) + 7) / 8);
            memcpy(seg.arg.data(), &args, sizeof(args));
            out.push_back(std::move(seg));
            list->has_segments = true;
            ex->log->add(3, "task list: launches %zu..%zu run as one persistent launch (fixed workspace)", i, j - 1);
            i = j;
            continue;
        }
        if (e != hipSuccess || hipMalloc(&d_table, table.size()) != hipSuccess) {
            for (size_t k = i; k < j; ++k) out.push_back(std::move(list->launches[k]));
            i = j;
            continue;
        }
        list->device_mem.push_back(d_table);
        if (hipMalloc(&d_ctl, sizeof(nce::PkCtl)) != hipSuccess || hipMemset(d_ctl, 0, sizeof(nce::PkCtl)) != hipSuccess || hipMemcpy(d_table, table.data(), table.size(), hipMemcpyHostToDevice) != hipSuccess) {
            for (size_t k = i; k < j; ++k) out.push_back(std::move(list->launches[k]));
            i = j;
            continue;
        }
        list->device_mem.push_back(d_ctl);
        nce::PkArgs args;
        args.layers = d_table;
        args.ctl = static_cast<nce::PkCtl*>(d_ctl);
        args.host_error = ex->pk_host_error;
        args.nlayers = (int32_t)(j - i);
        args.wait_us = (uint32_t)ex->opt.persistent_wait_us;
        seg.arg.resize((sizeof(args) + 7) / 8);
        memcpy(seg.arg.data(), &args, sizeof(args));
        out.push_back(std::move(seg));
        list->has_segments = true;
        ex->log->add(3, "task list: launches %zu..%zu run as one persistent launch", i, j - 1);
        i = j;
    }
    list->launches = std::move(out);
    return NCE_RESULT_SUCCESS;
}

}  // namespace

extern "C" {

nce_result_t nceGetVersion(uint32_t* major, uint32_t* minor) {
    if (major == nullptr || minor == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *major = NCE_HIP_VERSION_MAJOR;
    *minor = NCE_HIP_VERSION_MINOR;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceExecutorCreate(nce_executor_desc_t desc, nce_executor_handle_t* executor, nce_log_handle_t* log) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *executor = nullptr;
    if (log) *log = nullptr;
    nce_log_s* lg = new (std::nothrow) nce_log_s;
    nce_executor_s* ex = new (std::nothrow) nce_executor_s;
    if (lg == nullptr || ex == nullptr) {
        delete lg;
        delete ex;
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    }
    lg->level = desc.log_level;
    ex->log = lg;
    ex->device = desc.device_id;
    ex->opt = read_options();
    if (desc.device_id >= 0) {
        int count = 0;
        const hipError_t e = hipGetDeviceCount(&count);
        if (e != hipSuccess || desc.device_id >= count) {
            if (desc.log_level >= 1)
                fprintf(stderr, "nceExecutorCreate: no usable HIP device %d (%d visible): %s\n", desc.device_id, count,
                        hipGetErrorString(e));
            delete ex;
            delete lg;
            return NCE_RESULT_ERROR_UNSUPPORTED;
        }
        // The fixed workspace's address on this device (nceTaskListEnqueueNoAlloc); everything else works without it.
        if (hipSetDevice(desc.device_id) == hipSuccess) {
            // (persistent launches report through a pinned host word; made here, once, rather than by the first list that
            // needs it - lists of one executor may be prepared from several threads)
            if (ex->opt.persistent != 0 && hipHostMalloc(reinterpret_cast<void**>(&ex->pk_host_error), 64, hipHostMallocDefault) == hipSuccess)
                *ex->pk_host_error = 0;
            else
                ex->pk_host_error = nullptr;
            hipError_t we = nce::pk_workspace(desc.device_id, &ex->ws);
            if (we == hipSuccess) we = hipHostMalloc(reinterpret_cast<void**>(&ex->ws_staging), ex->ws.table_bytes, hipHostMallocDefault);
            if (we == hipSuccess) we = hipEventCreateWithFlags(&ex->ws_event, hipEventDisableTiming);
            ex->ws_ok = we == hipSuccess && desc.device_id < kWsMaxDevices;
            if (ex->ws_ok) ex->ws_failures_seen = ws_failures[desc.device_id].load();
            if (!ex->ws_ok) lg->add(2, "fixed workspace not available on device %d: %s", desc.device_id, hipGetErrorString(we));
        }
    }
    *executor = ex;
    if (log) *log = lg;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceExecutorDestroy(nce_executor_handle_t executor) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    delete executor->log;
    delete executor;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceClusterTaskValidate(nce_executor_handle_t executor, const nce_cluster_task_desc_t* task) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    try {
        Plan plan;
        return make_plan(executor->log, task, &plan);
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (...) {
        return NCE_RESULT_ERROR_UNKNOWN;
    }
}

nce_result_t nceClusterTaskEnqueue(nce_executor_handle_t executor, const nce_cluster_task_desc_t* task, void* hip_stream) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    try {
        Plan plan;
        const nce_result_t r = make_plan(executor->log, task, &plan);
        if (r != NCE_RESULT_SUCCESS) return r;
        if (executor->device < 0) {
            executor->log->add(1, "executor was created without a device (device_id < 0): it can validate, not launch");
            return NCE_RESULT_ERROR_UNSUPPORTED;
        }
        if (hipSetDevice(executor->device) != hipSuccess) return NCE_RESULT_ERROR_UNKNOWN;
        const ScopedLaunch ctx(&executor->opt, nullptr, executor->log);
        return launch_plan(executor, plan, static_cast<hipStream_t>(hip_stream));
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (...) {
        return NCE_RESULT_ERROR_UNKNOWN;
    }
}

nce_result_t nceTaskListCreate(nce_executor_handle_t executor, nce_task_list_handle_t* list) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (list == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *list = new (std::nothrow) nce_task_list_s;
    if (*list == nullptr) return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    (*list)->ex = executor;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceTaskListAppend(nce_task_list_handle_t list, const nce_cluster_task_desc_t* task) {
    if (list == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    try {
        Plan plan;
        const nce_result_t r = make_plan(list->ex->log, task, &plan);
        if (r != NCE_RESULT_SUCCESS) return r;
        std::lock_guard<std::mutex> lk(list->mu);
        list->plans.push_back(std::move(plan));
        list->drop_prepared();
        return NCE_RESULT_SUCCESS;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (...) {
        return NCE_RESULT_ERROR_UNKNOWN;
    }
}

namespace {

// Both enqueue forms. fixed_ws: nothing may be allocated or freed on the device - persistent segments (always tried in that
// form) keep their tables, counters and error word in the executor's fixed workspace.
nce_result_t enqueue_list(nce_task_list_handle_t list, void* hip_stream, bool fixed_ws) {
    if (list == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    nce_executor_s* const ex = list->ex;
    if (ex->device < 0) return NCE_RESULT_ERROR_UNSUPPORTED;
    if (hipSetDevice(ex->device) != hipSuccess) return NCE_RESULT_ERROR_UNKNOWN;
    const hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    try {
        std::lock_guard<std::mutex> lk(list->mu);
        if (fixed_ws) {
            // The form stages its layer tables through one pinned buffer and an event per executor: a captured copy would
            // re-read, at every replay, whatever list staged last, and an event recorded while capturing cannot be waited
            // for. So it is an eager-only entry point.
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
                ex->log->add(1, "nceTaskListEnqueueNoAlloc: the stream is being captured; this entry point cannot be recorded into a graph");
                return NCE_RESULT_ERROR_UNSUPPORTED;
            }
        }
        if (fixed_ws && !ex->ws_ok) {
            ex->log->add(1, "nceTaskListEnqueueNoAlloc: the fixed workspace was not found on device %d when the executor was created", ex->device);
            return NCE_RESULT_ERROR_UNSUPPORTED;
        }
        if (list->prepared && list->fixed_ws != fixed_ws) {
            if (fixed_ws && !list->device_mem.empty()) {
                // (switching forms would have to free what nceTaskListEnqueue allocated for this list)
                ex->log->add(1, "nceTaskListEnqueueNoAlloc: this list holds device allocations made by nceTaskListEnqueue; use one form per list");
                return NCE_RESULT_ERROR_INVALID_ARGUMENT;
            }
            list->drop_prepared();
        }
        if (list->prepared && list->has_segments && ex->pk_off.load()) list->drop_prepared();  // (the fixed form holds no device memory)
        if (!list->prepared) {
            // Kernel choice, grids and argument blocks are worked out once, here; later calls only replay them.
            list->drop_prepared();
            const bool persistent = (fixed_ws || ex->opt.persistent != 0) && !ex->pk_off.load();
            std::vector<PkAlt> alts;
            {
                const ScopedLaunch ctx(&ex->opt, &list->launches, ex->log);
                const nce_result_t r = run_plans(ex, list->plans, nullptr, persistent ? &alts : nullptr);
                if (r != NCE_RESULT_SUCCESS) {
                    list->launches.clear();
                    return r;
                }
            }
            if (persistent) {
                const ScopedLaunch ctx(&ex->opt, nullptr, ex->log);
                const nce_result_t r = build_segments(list, alts, fixed_ws);
                if (r != NCE_RESULT_SUCCESS) {
                    list->drop_prepared();
                    return r;
                }
            }
            list->fixed_ws = fixed_ws;
            list->prepared = true;
        }
        if (list->fixed_ws && list->has_segments) {
            // The workspace holds whatever the last list to use it left there: this list's tables go in ahead of its launches,
            // through the executor's pinned staging buffer (once the previous copy out of it has finished).
            std::lock_guard<std::mutex> ws_lock(ex->ws_mu);
            hipError_t e = ex->ws_event_pending ? hipEventSynchronize(ex->ws_event) : hipSuccess;
            if (e == hipSuccess) {
                memcpy(ex->ws_staging, list->ws_table.data(), list->ws_table.size());
                e = hipMemcpyAsync(ex->ws.table, ex->ws_staging, list->ws_table.size(), hipMemcpyHostToDevice, stream);
            }
            if (e == hipSuccess) {
                e = hipEventRecord(ex->ws_event, stream);
                ex->ws_event_pending = e == hipSuccess;
            }
            if (e != hipSuccess) {
                ex->log->add(1, "copy of the layer tables to the fixed workspace failed: %s", hipGetErrorString(e));
                return NCE_RESULT_ERROR_UNKNOWN;
            }
            ex->ws_used.store(true);
        }
        for (const nce::RecordedLaunch& l : list->launches) {
            const hipError_t e = nce::replay(l, stream);
            if (e != hipSuccess) {
                ex->log->add(1, "kernel launch failed: %s", hipGetErrorString(e));
                return NCE_RESULT_ERROR_UNKNOWN;
            }
        }
        return NCE_RESULT_SUCCESS;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (...) {
        return NCE_RESULT_ERROR_UNKNOWN;
    }
}

}  // namespace

nce_result_t nceTaskListEnqueue(nce_task_list_handle_t list, void* hip_stream) {
    return enqueue_list(list, hip_stream, false);
}

nce_result_t nceTaskListEnqueueNoAlloc(nce_task_list_handle_t list, void* hip_stream) {
    return enqueue_list(list, hip_stream, true);
}

nce_result_t nceTaskListDestroy(nce_task_list_handle_t list) {
    if (list == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    delete list;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceExecutorSynchronize(nce_executor_handle_t executor, void* hip_stream) {
    if (executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (executor->device < 0) return NCE_RESULT_ERROR_UNSUPPORTED;
    if (hipSetDevice(executor->device) != hipSuccess) return NCE_RESULT_ERROR_UNKNOWN;
    const hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) {
        executor->log->add(1, "synchronize failed: %s", hipGetErrorString(e));
        return NCE_RESULT_ERROR_UNKNOWN;
    }
    uint32_t code = 0;
    if (executor->pk_host_error != nullptr && *executor->pk_host_error != 0) {
        code = *executor->pk_host_error;
        *executor->pk_host_error = 0;
    }
    if (executor->ws_used.load()) {  // (the fixed workspace's error word lives in device memory)
        uint32_t ws_code = 0;
        if (hipMemcpy(&ws_code, executor->ws.error, sizeof(ws_code), hipMemcpyDeviceToHost) == hipSuccess && ws_code != 0) {
            // (a launch that gave up leaves the workspace's counters between multiples of 32)
            (void)hipMemset(executor->ws.error, 0, sizeof(ws_code));
            (void)hipMemset(executor->ws.ctl, 0, sizeof(nce::PkCtl));
            code = std::max(code, ws_code);
            ws_failures[executor->device].fetch_add(1);
        }
        // (another executor of this device may have read and cleared the word first: its launches share the counters
        // with ours, so a failure it found leaves this executor's outputs in doubt as well)
        const uint32_t failures = ws_failures[executor->device].load();
        if (failures != executor->ws_failures_seen) {
            executor->ws_failures_seen = failures;
            code = std::max<uint32_t>(code, 1);
        }
    }
    if (code != 0) {
        // A persistent segment gave up (a bounded wait ran out, or its workgroups were not placed as expected): what it
        // wrote is incomplete. Persistent launches are off for this executor from here on; the caller re-enqueues.
        executor->log->add(1, "a persistent task-list launch did not complete (code %u); its outputs are invalid, persistent launches are now off", code);
        executor->pk_off.store(true);
        return NCE_RESULT_ERROR_UNKNOWN;
    }
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceLogHandleGetString(nce_log_handle_t log, size_t* size, char* buf) {
    if (log == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (size == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lk(log->mu);
    if (buf == nullptr) {
        *size = log->text.size() + 1;
        return NCE_RESULT_SUCCESS;
    }
    if (*size == 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    const size_t n = std::min(*size - 1, log->text.size());
    memcpy(buf, log->text.data(), n);
    buf[n] = '\0';
    *size = n + 1;
    log->text.clear();
    return NCE_RESULT_SUCCESS;
}

}  // extern "C"
