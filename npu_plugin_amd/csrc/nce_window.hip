// DWCONV, AVEPOOL and MAXPOOL tasks: per-channel sliding-window ops on NHWC activations.
// Semantics (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc):
//   DWCONV  :834-945   acc = sum (a - zp_a) * (w - zp_w) over in-image taps, scale/bias from the table
//   AVEPOOL :1805-1905 acc = sum (a - zp_a) over in-image taps (window weight 1, :907-913), the
//                      1/(KY*KX) lives in the PPE scale
//   MAXPOOL :1759-1803 max of the raw values, scale 1 / shift 0 / zero point 0, clamp only
// Depthwise weights are one 16-byte-multiple row per channel holding the KY*KX taps row-major
// (src/vpux_compiler/src/dialect/VPU/utils/const_utils.cpp:101-120,216-243).
//
// Memory-bound: a lane owns one 16-channel group (one 128-bit load per tap) of one output pixel;
// adjacent lanes own adjacent channel groups, so a wavefront reads whole NHWC pixels contiguously.
#include "nce_ppe_device.h"

namespace nce {
namespace {

enum { MODE_DW = 0, MODE_AVG = 1, MODE_MAX = 2 };

constexpr int SLAB_GROUPS = 16;                  // channel groups (of 16) one block works on
constexpr int SLAB_CH = SLAB_GROUPS * 16;        // 256 channels

template <bool SIGNED>
__device__ __forceinline__ int32_t byte_at(uint32_t w, int i) {
    return SIGNED ? (int32_t)(int8_t)(w >> (8 * i)) : (int32_t)((w >> (8 * i)) & 0xFFu);
}

template <int MODE, bool A_SIGNED, bool W_SIGNED>
__global__ __launch_bounds__(256) void window_kernel(TaskDev t, Box box, int64_t npix, int items_per_thread) {
    extern __shared__ uint8_t s_w[];  // MODE_DW: [tap][SLAB_CH] weight bytes of this block's channel slab

    const int32_t cgroups = box.bc >> 4;
    const int32_t slab0 = blockIdx.y * SLAB_GROUPS;  // first channel group of the slab
    const int32_t nslab = min(SLAB_GROUPS, cgroups - slab0);
    const int ntaps = t.ky * t.kx;

    if (MODE == MODE_DW) {
        // transpose [channel][tap] rows into [tap][channel]
        for (int ch = threadIdx.x; ch < nslab * 16; ch += blockDim.x) {
            const uint8_t* row = t.weights + (int64_t)(box.z0 + slab0 * 16 + ch) * t.w_stride_oc;
            for (int tap = 0; tap < ntaps; ++tap) s_w[tap * SLAB_CH + ch] = row[tap];
        }
        __syncthreads();
    }

    const int64_t nitems = npix * nslab;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x * items_per_thread;
    for (int it = 0; it < items_per_thread; ++it) {
        const int64_t item = first + (int64_t)it * blockDim.x + threadIdx.x;
        if (item >= nitems) break;
        const int32_t cg = (int32_t)(item % nslab);
        int64_t r = item / nslab;
        const int32_t bx = (int32_t)(r % box.bw);
        r /= box.bw;
        const int32_t by = (int32_t)(r % box.bh);
        const int64_t n = r / box.bh;
        const int32_t oc = box.z0 + ((slab0 + cg) << 4);
        const int32_t oy = box.y0 + by, ox = box.x0 + bx;
        const int32_t iy0 = oy * t.sy - t.pt, ix0 = ox * t.sx - t.pl;
        const uint8_t* src = t.in.data + n * t.in.sn + oc;

        int32_t acc[16];
        const int32_t init = MODE == MODE_MAX ? (A_SIGNED ? -128 : 0) : 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = init;

        for (int ky = 0; ky < t.ky; ++ky) {
            const int32_t iy = iy0 + ky;
            if (iy < 0 || iy >= t.in.h) continue;
            for (int kx = 0; kx < t.kx; ++kx) {
                const int32_t ix = ix0 + kx;
                if (ix < 0 || ix >= t.in.w) continue;
                const uint4 va = *reinterpret_cast<const uint4*>(src + (int64_t)iy * t.in.sh + (int64_t)ix * t.in.sw);
                const uint32_t wa[4] = {va.x, va.y, va.z, va.w};
                if (MODE == MODE_DW) {
                    const uint4 vw = *reinterpret_cast<const uint4*>(s_w + (ky * t.kx + kx) * SLAB_CH + (cg << 4));
                    const uint32_t ww[4] = {vw.x, vw.y, vw.z, vw.w};
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        acc[i] += (byte_at<A_SIGNED>(wa[i >> 2], i & 3) - t.in.zp) *
                                  (byte_at<W_SIGNED>(ww[i >> 2], i & 3) - t.w_zp);
                } else if (MODE == MODE_AVG) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[i] += byte_at<A_SIGNED>(wa[i >> 2], i & 3) - t.in.zp;
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[i] = max(acc[i], byte_at<A_SIGNED>(wa[i >> 2], i & 3));
                }
            }
        }

        uint32_t wo[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int32_t y;
            if (MODE == MODE_MAX) {
                y = acc[i] < t.ppe.lo ? t.ppe.lo : (acc[i] > t.ppe.hi ? t.ppe.hi : acc[i]);
            } else {
                int32_t mult = t.ppe.quant_mult, shift = t.ppe.quant_shift, bias = 0;
                if (t.table != nullptr) {
                    const int32_t* row = t.table + (int64_t)(oc + i) * t.table_stride;
                    mult = table_mult(row[2]);
                    shift = table_shift(row[2]);
                    bias = row[3];
                }
                y = ppe_apply(acc[i], bias, mult, shift, t.ppe);
            }
            wo[i >> 2] |= ((uint32_t)y & 0xFFu) << (8 * (i & 3));
        }
        *reinterpret_cast<uint4*>(t.out.data + n * t.out.sn + (int64_t)oy * t.out.sh + (int64_t)ox * t.out.sw + oc) =
                make_uint4(wo[0], wo[1], wo[2], wo[3]);
    }
}

template <int MODE>
hipError_t launch_window(const TaskDev& t, const Box& box, hipStream_t s) {
    const int64_t npix = (int64_t)t.out.n * box.bh * box.bw;
    const int32_t cgroups = box.bc >> 4;
    if (npix == 0 || cgroups == 0) return hipSuccess;
    const int nslabs = (cgroups + SLAB_GROUPS - 1) / SLAB_GROUPS;
    const int64_t items = npix * (cgroups < SLAB_GROUPS ? cgroups : SLAB_GROUPS);
    const int ipt = items > (int64_t)256 * 4096 ? 4 : 1;
    const int64_t blocks = (items + 256 * ipt - 1) / (256 * ipt);
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const size_t lds = MODE == MODE_DW ? (size_t)t.ky * t.kx * SLAB_CH : 0;
    const dim3 grid((unsigned)blocks, (unsigned)nslabs);
    const int sel = (t.in.is_signed ? 2 : 0) | (t.w_is_signed ? 1 : 0);
    switch (sel) {
    case 0: hipLaunchKernelGGL((window_kernel<MODE, false, false>), grid, dim3(256), lds, s, t, box, npix, ipt); break;
    case 1: hipLaunchKernelGGL((window_kernel<MODE, false, true>), grid, dim3(256), lds, s, t, box, npix, ipt); break;
    case 2: hipLaunchKernelGGL((window_kernel<MODE, true, false>), grid, dim3(256), lds, s, t, box, npix, ipt); break;
    default: hipLaunchKernelGGL((window_kernel<MODE, true, true>), grid, dim3(256), lds, s, t, box, npix, ipt); break;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_pool(const TaskDev& t, const Box& box, bool is_max, hipStream_t stream) {
    return is_max ? launch_window<MODE_MAX>(t, box, stream) : launch_window<MODE_AVG>(t, box, stream);
}

hipError_t launch_dwconv(const TaskDev& t, const Box& box, hipStream_t stream) {
    return launch_window<MODE_DW>(t, box, stream);
}

}  // namespace nce
