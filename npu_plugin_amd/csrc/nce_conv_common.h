// Shared pieces of the CONV kernels: launch arguments, MFMA operand types and the fused PPE store.
#pragma once

#include "nce_ppe_device.h"

namespace nce {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Division of a 31-bit value by a run-time constant as multiply-high + shift (host-prepared):
// m = ceil(2^(31+s) / d) with s = ceil(log2 d); q = umulhi(n, m) >> (s - 1). Exact for n < 2^31.
struct FastDiv {
    uint32_t d, m, sh;  // m == 0: d == 1
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    f.m = 0;
    f.sh = 0;
    if (d > 1) {
        uint32_t s = 0;
        while ((1ull << s) < d) ++s;
        f.m = (uint32_t)(((1ull << (31 + s)) + d - 1) / d);
        f.sh = s - 1;
    }
    return f;
}

// (F: FastDiv in any address space)
template <typename F>
__device__ __forceinline__ uint32_t fdiv(uint32_t n, const F& f) {
    return f.m == 0 ? n : (__umulhi(n, f.m) >> f.sh);
}

// A copy, in registers, of a struct that may live in the constant address space.
template <typename T, typename S>
__device__ __forceinline__ T generic_copy(const S& src) {
    T t;
    __builtin_memcpy(&t, &src, sizeof(T));
    return t;
}

struct ConvArgs {
    const uint8_t* in;
    int64_t in_sn, in_sh, in_sw;
    int32_t H, W, IC;
    const uint8_t* w;
    int64_t w_soc;
    const int32_t* table;
    int64_t table_stride;
    uint8_t* out;
    int64_t out_sn, out_sh, out_sw, out_sc;
    int32_t x0, y0, z0, bw, bh, bc;
    int32_t M;  // pixels in the box over all batches (< 2^31)
    FastDiv div_bw, div_bh, div_pitch, div_rows_full;
    int32_t KY, KX, SY, SX, PT, PL;
    int32_t KG;   // 16-byte groups along K: KY*KX*IC/16
    int32_t ICG;  // 16-byte groups per tap: IC/16
    uint32_t a_xor, w_xor;  // 0x80808080 for u8 storage, 0 for i8
    uint32_t fill;          // out-of-image activation word, re-biased
    uint32_t fill_raw;      // the same byte as stored (the input zero point), 0..255
    int32_t da, dw;         // (storage offset - zero point) of activations / weights
    int32_t ktot;           // KY*KX*IC
    // halo kernel only
    int32_t pitchpx;     // staged pixels per input row: W + pad_left + pad_right
    int32_t nslots_max;  // input rows one tile may stage
    int32_t rows_max;    // output rows one tile may touch
    int32_t nchunks;     // 64-byte chunks along IC
    int32_t halo_bytes;  // nslots_max * pitchpx * 64
    PpeDev ppe;
};

__device__ __forceinline__ int32_t bytesum(uint4 v) {
    int32_t s = 0;
    s = __builtin_amdgcn_sdot4((int)v.x, 0x01010101, s, false);
    s = __builtin_amdgcn_sdot4((int)v.y, 0x01010101, s, false);
    s = __builtin_amdgcn_sdot4((int)v.z, 0x01010101, s, false);
    s = __builtin_amdgcn_sdot4((int)v.w, 0x01010101, s, false);
    return s;
}

// MFMA row i of the weight operand carries channel chan_of_row(i) of its 32-channel fragment, so
// that the 16 accumulator registers of a lane (rows 8*(v/4) + 4*half + v%4) are 16 CONSECUTIVE
// channels 16*half .. 16*half+15 and one 128-bit store writes them.
__device__ __forceinline__ int chan_of_row(int i) {
    return 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
}
__device__ __forceinline__ int row_of_chan(int c) {
    return 8 * ((c >> 2) & 3) + 4 * (c >> 4) + (c & 3);
}

// Per-channel epilogue constants in LDS (BN entries each).
struct EpiSmem {
    double* M;
    double* B;
    int32_t* w2;
    int32_t* bias;
    int32_t* corr;
    int32_t* wsum;
};

// Load the weight-table rows of this workgroup's channels. Call before the main loop (all threads).
__device__ __forceinline__ void epi_load_table(const ConvArgs& a, const EpiSmem& s, int tid, int nthreads, int bn,
                                               int32_t oc0, int32_t noc) {
    for (int c = tid; c < bn; c += nthreads) {
        int32_t w2 = 0, b = 0;
        if (c < noc) {
            const int32_t* row = a.table + (int64_t)(oc0 + c) * a.table_stride;
            w2 = row[2];
            b = row[3];
        }
        s.w2[c] = w2;
        s.bias[c] = b;
        s.wsum[c] = 0;
    }
}

// After the main loop (wsum complete, behind a barrier): FP64 constants per channel and the PPE
// specialisation the whole workgroup runs.
__device__ __forceinline__ int epi_constants(const ConvArgs& a, const EpiSmem& s, int tid, int nthreads, int bn,
                                             PpeF64* pu) {
    int bad_shift = 0, small_shift = 0;
    for (int c = tid; c < bn; c += nthreads) {
        const int32_t w2 = s.w2[c];
        const int32_t shift = table_shift(w2);
        bad_shift |= shift > kMaxF64Shift;
        // |acc| <= K * 255 * 255 (and never beyond int32: the accumulator wraps)
        const int64_t acc_bound = min((int64_t)a.ktot * 65025, (int64_t)2147483648LL);
        small_shift |= ppe_may_saturate(acc_bound, s.bias[c], table_mult(w2), shift);
    }
    const bool use_int = __syncthreads_or(bad_shift) != 0;
    const bool may_sat = __syncthreads_or(small_shift) != 0;
    *pu = ppe_f64_setup(a.ppe, may_sat);
    const int mode = ppe_mode_of(*pu, use_int);
    for (int c = tid; c < bn; c += nthreads) {
        const int32_t w2 = s.w2[c];
        const int32_t mult = table_mult(w2), shift = table_shift(w2);
        const int32_t corr = a.da * s.wsum[c];  // |da| <= 255, |sum w'| < 2^23
        const double M = ppe_scale_M(mult, shift);
        s.M[c] = M;
        s.B[c] = ppe_mode_B(__builtin_fma((double)corr, M, ppe_scale_B(s.bias[c], M, shift, a.ppe.round_mode)), mode, *pu);
        s.corr[c] = corr;
    }
    __syncthreads();
    return mode;
}

// PPE + store of one wavefront's accumulators: AF channel fragments x BF pixel fragments.
//   ocw     first channel (workgroup-local) of this wave's fragment 0
//   dst[x]  output address of this lane's pixel of fragment x at workgroup channel 0 (valid[x] says
//           whether that pixel exists)
//   acorr   per-pixel accumulator correction (weights zero point); ACORR = false: not used
template <int AF, int BF, int MODE, bool ACORR>
__device__ __forceinline__ void epi_store_mode(const ConvArgs& a, const EpiSmem& s, v16i (&acc)[AF][BF], int ocw, int noc,
                                               int half, uint8_t* const (&dst)[BF], const bool (&valid)[BF],
                                               const int32_t (&acorr)[BF], const PpeF64& pu) {
#pragma unroll
    for (int f = 0; f < AF; ++f) {
        const int ocl = ocw + 32 * f + 16 * half;
        if (ocl >= noc) continue;
        uint32_t wo[BF][4];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int c = ocl + v;
            double M = 0.0, B = 0.0;
            int32_t w2 = 0, bias = 0, corr = 0;
            if (MODE == PPE_MODE_INT) {
                w2 = s.w2[c];
                bias = s.bias[c];
                corr = s.corr[c];
            } else {
                M = s.M[c];
                B = s.B[c];
            }
#pragma unroll
            for (int x = 0; x < BF; ++x) {
                int32_t av = acc[f][x][v];
                if (ACORR) av = (int32_t)((uint32_t)av + (uint32_t)acorr[x]);
                int32_t y;
                if (MODE == PPE_MODE_INT)
                    y = ppe_apply((int32_t)((uint32_t)av + (uint32_t)corr), bias, table_mult(w2), table_shift(w2), a.ppe);
                else
                    y = ppe_finish_mode<MODE>(__builtin_fma((double)av, M, B), pu);
                const uint32_t b = (uint32_t)y & 0xFFu;
                wo[x][v >> 2] = (v & 3) == 0 ? b : (wo[x][v >> 2] | (b << (8 * (v & 3))));
            }
        }
#pragma unroll
        for (int x = 0; x < BF; ++x)
            if (valid[x]) store_channels16(dst[x] + ocl * a.out_sc, a.out_sc, wo[x][0], wo[x][1], wo[x][2], wo[x][3]);
    }
}

template <int AF, int BF, bool ACORR>
__device__ __forceinline__ void epi_store(const ConvArgs& a, const EpiSmem& s, v16i (&acc)[AF][BF], int ocw, int noc,
                                          int half, uint8_t* const (&dst)[BF], const bool (&valid)[BF],
                                          const int32_t (&acorr)[BF], int mode, const PpeF64& pu) {
    if (mode == PPE_MODE_FOLDED) epi_store_mode<AF, BF, PPE_MODE_FOLDED, ACORR>(a, s, acc, ocw, noc, half, dst, valid, acorr, pu);
    else if (mode == PPE_MODE_SLOPE) epi_store_mode<AF, BF, PPE_MODE_SLOPE, ACORR>(a, s, acc, ocw, noc, half, dst, valid, acorr, pu);
    else epi_store_mode<AF, BF, PPE_MODE_INT, ACORR>(a, s, acc, ocw, noc, half, dst, valid, acorr, pu);
}

hipError_t launch_conv_gather(const ConvArgs& a, hipStream_t stream);
// Returns hipErrorNotSupported when the shape does not fit the halo kernel (caller falls back).
hipError_t launch_conv_halo(const ConvArgs& a, hipStream_t stream);
// allow_chunked: also take reductions longer than one LDS slice (weights staged chunk by chunk)
// A residual add fused into the epilogue of the convolution that produces one of its inputs (task lists: a
// convolution directly followed by an ELTWISE task reading its output). The convolution's own output is still
// written; the add's output is computed from the stored bytes, so both tensors hold what the two tasks give.
// All three tensors of the add are dense NHWC of the convolution's output shape: element offsets coincide.
struct FuseAdd {
    const uint8_t* other;  // the add's other input
    uint8_t* out;          // the add's output
    uint32_t mults;        // input multiplier of the convolution's value | of the other input << 16
    uint32_t in_flip;      // 0x80808080 for signed inputs (they enter the 16-bit dot product 128 higher)
    int32_t c0h;           // -(mults . zero points), less 128 * (sum of multipliers) for signed inputs
    int32_t mq;            // quant_mult * 2^(32 - shift)
    int64_t cq;            // (2^(shift-1) + zero point * 2^shift) * 2^(32 - shift)
    int32_t ilo, ihi;      // clamp bounds (signed outputs 128 higher)
    uint32_t flip;         // 0x80808080 for signed outputs
};

// fuse: optional; hipErrorNotSupported when the kernel variant that would run the task cannot carry the add.
hipError_t launch_conv_wres(const ConvArgs& a, hipStream_t stream, bool allow_chunked, const FuseAdd* fuse = nullptr);
// LDS-tiled kernel for many output channels; shape 1.. selects a tile shape (see nce_conv_tiled.hip), 0 the automatic choice.
hipError_t launch_conv_tiled(const ConvArgs& a, hipStream_t stream, int shape, const FuseAdd* fuse = nullptr);
// Patch kernel for kernels larger than 1x1 at stride 1: weights slice and the patch's input pixels (with halo) both in LDS.
// nf = 0 / pr = 0 / waves = 0: automatic channel fragments per slice (2 or 4) / output rows per patch / waves per workgroup (8, 16);
// npx = 1 (with 16 waves): one pixel fragment per wave and group instead of two.
hipError_t launch_conv_patch(const ConvArgs& a, hipStream_t stream, int nf, int pr, int waves, int npx);

}  // namespace nce
