// ELTWISE add task: out = PPE(in1_mult * (a - zp_a) + in2_mult * (b - zp_b)).
// Semantics: src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:1541-1555
// (per-input multipliers elop_scale_a/b) and :1651-1757 (scale override from the PPE task).
//
// Memory-bound: each lane moves one 16-byte channel group of both inputs and of the output
// (global_load_dwordx4 x2, global_store_dwordx4 x1), 48 algorithmic bytes per 16 outputs.
#include "nce_ppe_device.h"

namespace nce {
namespace {

template <bool SIGNED>
__device__ __forceinline__ int32_t byte_at(uint32_t w, int i) {
    return SIGNED ? (int32_t)(int8_t)(w >> (8 * i)) : (int32_t)((w >> (8 * i)) & 0xFFu);
}

template <bool FLAT, bool HAS_TABLE, bool A_SIGNED, bool B_SIGNED>
__global__ __launch_bounds__(256) void eltwise_kernel(TaskDev t, Box box, int64_t nchunks) {
    const int32_t cgroups = box.bc >> 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < nchunks;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t off_a, off_b, off_o;
        int32_t oc;
        if (FLAT) {
            off_a = off_b = off_o = idx << 4;
            oc = (int32_t)(idx % cgroups) << 4;
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
            off_o = n * t.out.sn + y * t.out.sh + x * t.out.sw + oc;
        }
        const uint4 va = *reinterpret_cast<const uint4*>(t.in.data + off_a);
        const uint4 vb = *reinterpret_cast<const uint4*>(t.in2.data + off_b);
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w};
        const uint32_t wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t wo[4];
        // c0 folds both zero points: m1*(a-zpa) + m2*(b-zpb) = m1*a + m2*b + c0. |c0| < 2^26.
        const int32_t c0 = -(t.ppe.in1_mult * t.in.zp + t.ppe.in2_mult * t.in2.zp);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t packed = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int32_t a = byte_at<A_SIGNED>(wa[d], i);
                const int32_t b = byte_at<B_SIGNED>(wb[d], i);
                const int32_t acc = t.ppe.in1_mult * a + t.ppe.in2_mult * b + c0;
                int32_t mult = t.ppe.quant_mult, shift = t.ppe.quant_shift, bias = 0;
                if (HAS_TABLE) {
                    const int32_t* row = t.table + (int64_t)(oc + 4 * d + i) * t.table_stride;
                    mult = table_mult(row[2]);
                    shift = table_shift(row[2]);
                    bias = row[3];
                }
                const int32_t y = ppe_apply(acc, bias, mult, shift, t.ppe);
                packed |= ((uint32_t)y & 0xFFu) << (8 * i);
            }
            wo[d] = packed;
        }
        *reinterpret_cast<uint4*>(t.out.data + off_o) = make_uint4(wo[0], wo[1], wo[2], wo[3]);
    }
}

bool is_dense_nhwc(const TensorDev& x) {
    return x.sw == x.c && x.sh == (int64_t)x.w * x.c && x.sn == (int64_t)x.h * x.w * x.c;
}

template <bool FLAT, bool HAS_TABLE>
void launch_signed(const TaskDev& t, const Box& box, int64_t nchunks, int grid, hipStream_t s) {
    const int sel = (t.in.is_signed ? 2 : 0) | (t.in2.is_signed ? 1 : 0);
    switch (sel) {
    case 0: hipLaunchKernelGGL((eltwise_kernel<FLAT, HAS_TABLE, false, false>), dim3(grid), dim3(256), 0, s, t, box, nchunks); break;
    case 1: hipLaunchKernelGGL((eltwise_kernel<FLAT, HAS_TABLE, false, true>), dim3(grid), dim3(256), 0, s, t, box, nchunks); break;
    case 2: hipLaunchKernelGGL((eltwise_kernel<FLAT, HAS_TABLE, true, false>), dim3(grid), dim3(256), 0, s, t, box, nchunks); break;
    default: hipLaunchKernelGGL((eltwise_kernel<FLAT, HAS_TABLE, true, true>), dim3(grid), dim3(256), 0, s, t, box, nchunks); break;
    }
}

}  // namespace

hipError_t launch_eltwise(const TaskDev& t, const Box& box, hipStream_t stream) {
    const int64_t nchunks = (int64_t)t.out.n * box.bh * box.bw * (box.bc >> 4);
    if (nchunks == 0) return hipSuccess;
    const bool full = box.x0 == 0 && box.y0 == 0 && box.z0 == 0 && box.bw == t.out.w && box.bh == t.out.h &&
                      box.bc == t.out.c;
    const bool flat = full && is_dense_nhwc(t.in) && is_dense_nhwc(t.in2) && is_dense_nhwc(t.out);
    const bool has_table = t.table != nullptr;
    int64_t blocks = (nchunks + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    const int grid = (int)blocks;
    if (flat) {
        if (has_table) launch_signed<true, true>(t, box, nchunks, grid, stream);
        else launch_signed<true, false>(t, box, nchunks, grid, stream);
    } else {
        if (has_table) launch_signed<false, true>(t, box, nchunks, grid, stream);
        else launch_signed<false, false>(t, box, nchunks, grid, stream);
    }
    return hipGetLastError();
}

}  // namespace nce
