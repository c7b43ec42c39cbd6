// CONV task (ZMajor: NHWC activations, OYXI weights) as an implicit GEMM on the gfx950 matrix
// cores: D[oc][pixel] += W[oc][k] * A[pixel][k], k = (ky, kx, ic) with ic innermost - the order
// both tensors already have in memory, so a 16-byte MFMA operand is 16 consecutive input channels
// of one tap. v_mfma_i32_32x32x32_i8 accumulates in int32; the PPE runs on the accumulators in
// registers and each lane stores 16 consecutive output channels of one pixel with one 128-bit store.
//
// Semantics: src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc
//   :834-882  activations: zero point removed before the MAC (mpe_actbias), padding contributes 0
//   :884-945  weights: zero point removed (mpe_wtbias)
//   :1952-2045 PPE scale from the weight table (ppe_scale_override = 0 for CONV)
//
// The matrix cores multiply signed bytes. u8 operands are re-biased by 128 (x ^ 0x80) and the
// difference between 128 and the real zero point is restored exactly in the epilogue:
//   sum (a-zpa)(w-zpw) = sum a'w' + da * sum w' + dw * (sum a' + K*da),  a' = a-offa, da = offa-zpa ...
// Out-of-image taps are filled with the byte zp_a, so that (a' + da) = 0 there.
#include "nce_conv_common.h"

namespace nce {
namespace {

constexpr int BN = 64;    // output channels per workgroup
constexpr int ROW = 80;   // LDS row pitch: 64 bytes of K + 16 bytes of padding against bank conflicts
constexpr int NTHREADS = 256;

// PXF = 32-pixel fragments per wavefront; the workgroup tile is (4 * 32 * PXF) pixels x 64 channels.
template <int PXF>
__global__ __launch_bounds__(NTHREADS) void conv_igemm_kernel(ConvArgs a) {
    prefetch_kernel_arguments<sizeof(ConvArgs)>();
    constexpr int BM = 128 * PXF;
    constexpr int NB = 2 * PXF;  // activation rows each thread stages per step

    __shared__ __attribute__((aligned(16))) uint8_t sA[2][BN * ROW];
    __shared__ __attribute__((aligned(16))) uint8_t sB[2][BM * ROW];
    __shared__ int32_t sW2[BN], sBias[BN], sWsum[BN], sCorr[BN];
    __shared__ double sM[BN], sBc[BN];
    __shared__ int32_t sAsum[BM];
    const EpiSmem es = {sM, sBc, sW2, sBias, sCorr, sWsum};

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int half = lane >> 5;
    const int l32 = lane & 31;

    const uint32_t ntiles = ((uint32_t)a.M + BM - 1) / BM;
    const uint32_t tile = xcd_tile(blockIdx.x, ntiles);
    if (tile >= ntiles) return;  // uniform for the whole workgroup
    const int32_t m0 = tile * BM;
    const int32_t oc0 = a.z0 + blockIdx.y * BN;
    const int32_t noc = min(BN, a.z0 + a.bc - oc0);

    epi_load_table(a, es, tid, NTHREADS, BN, oc0, noc);
    for (int i = tid; i < BM; i += NTHREADS) sAsum[i] = 0;

    // ---- staging assignment: thread -> (row, 16-byte group) -------------------------------
    const int grp = tid & 3;
    const int srow = tid >> 2;  // 0..63
    const bool w_valid = srow < noc;
    const uint8_t* w_ptr = a.w + (int64_t)(oc0 + srow) * a.w_soc;

    const uint8_t* b_base[NB];
    int32_t b_iy0[NB], b_ix0[NB];
    bool b_valid[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int32_t p = m0 + srow + 64 * i;
        b_valid[i] = p < a.M;
        const int32_t pp = b_valid[i] ? p : 0;
        const int32_t rr = fdiv(pp, a.div_bw);
        const int32_t bx = pp - rr * a.bw;
        const int32_t n = fdiv(rr, a.div_bh);
        const int32_t by = rr - n * a.bh;
        b_base[i] = a.in + (int64_t)n * a.in_sn;
        b_iy0[i] = (a.y0 + by) * a.SY - a.PT;
        b_ix0[i] = (a.x0 + bx) * a.SX - a.PL;
    }

    // position of this thread's group inside K: g = step*4 + grp -> (ky, kx, icg)
    int32_t g = grp;
    int32_t icg = grp, kx = 0, ky = 0;
    while (icg >= a.ICG) {
        icg -= a.ICG;
        if (++kx == a.KX) {
            kx = 0;
            ++ky;
        }
    }

    uint4 regA;
    uint4 regB[NB];
    int32_t wsum = 0;
    int32_t asum[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) asum[i] = 0;
    const uint4 fill4 = make_uint4(a.fill, a.fill, a.fill, a.fill);

    auto load_step = [&]() {
        const bool g_valid = g < a.KG;
        regA = make_uint4(0, 0, 0, 0);
        if (g_valid && w_valid) {
            regA = *reinterpret_cast<const uint4*>(w_ptr + (int64_t)g * 16);
            regA.x ^= a.w_xor;
            regA.y ^= a.w_xor;
            regA.z ^= a.w_xor;
            regA.w ^= a.w_xor;
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int32_t iy = b_iy0[i] + ky;
            const int32_t ix = b_ix0[i] + kx;
            const bool inb = g_valid && b_valid[i] && (uint32_t)iy < (uint32_t)a.H && (uint32_t)ix < (uint32_t)a.W;
            uint4 v = fill4;
            if (inb) {
                v = *reinterpret_cast<const uint4*>(b_base[i] + (int64_t)iy * a.in_sh + (int64_t)ix * a.in_sw +
                                                    (icg << 4));
                v.x ^= a.a_xor;
                v.y ^= a.a_xor;
                v.z ^= a.a_xor;
                v.w ^= a.a_xor;
            }
            regB[i] = v;
        }
        if (a.da != 0) wsum += bytesum(regA);
        if (a.dw != 0 && g_valid) {
#pragma unroll
            for (int i = 0; i < NB; ++i) asum[i] += bytesum(regB[i]);
        }
        // advance to the next step's group
        g += 4;
        icg += 4;
        while (icg >= a.ICG) {
            icg -= a.ICG;
            if (++kx == a.KX) {
                kx = 0;
                ++ky;
            }
        }
    };
    auto store_step = [&](int buf) {
        *reinterpret_cast<uint4*>(&sA[buf][srow * ROW + grp * 16]) = regA;
#pragma unroll
        for (int i = 0; i < NB; ++i)
            *reinterpret_cast<uint4*>(&sB[buf][(srow + 64 * i) * ROW + grp * 16]) = regB[i];
    };

    // ---- accumulators ------------------------------------------------------------------------
    v16i acc[2][PXF];
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int x = 0; x < PXF; ++x)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[f][x][v] = 0;

    // MFMA row i of the weight operand carries channel 16*((i>>2)&1) + 4*(i>>3) + (i&3), so that the
    // 16 accumulator registers of a lane are 16 CONSECUTIVE channels (16*half .. 16*half+15).
    const int a_row = chan_of_row(l32);
    const int b_row0 = wave * 32 * PXF + l32;

    const int nsteps = (a.KG + 3) >> 2;
    load_step();
    store_step(0);
    __syncthreads();
    for (int step = 0; step < nsteps; ++step) {
        const int buf = step & 1;
        const bool more = step + 1 < nsteps;
        if (more) load_step();
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int koff = (kk * 2 + half) * 16;
            v4i fa[2], fb[PXF];
#pragma unroll
            for (int f = 0; f < 2; ++f) fa[f] = *reinterpret_cast<const v4i*>(&sA[buf][(32 * f + a_row) * ROW + koff]);
#pragma unroll
            for (int x = 0; x < PXF; ++x) fb[x] = *reinterpret_cast<const v4i*>(&sB[buf][(b_row0 + 32 * x) * ROW + koff]);
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int x = 0; x < PXF; ++x)
                    acc[f][x] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[f], fb[x], acc[f][x], 0, 0, 0);
        }
        if (more) store_step(buf ^ 1);
        __syncthreads();
    }

    // ---- per-channel epilogue constants ------------------------------------------------------
    // Zero-point corrections (only when a zero point differs from the storage offset): the
    // weight-sum term is constant per channel and goes into B; the activation-sum term is per pixel.
    if (a.da != 0 || a.dw != 0) {
        if (a.da != 0) atomicAdd(&sWsum[srow], wsum);
        if (a.dw != 0) {
#pragma unroll
            for (int i = 0; i < NB; ++i) atomicAdd(&sAsum[srow + 64 * i], asum[i]);
        }
        __syncthreads();
    }
    PpeF64 pu;
    const int mode = epi_constants(a, es, tid, NTHREADS, BN, &pu);

    // ---- PPE + store -----------------------------------------------------------------------------
    uint8_t* dst[PXF];
    int32_t a_corr[PXF];
    bool p_valid[PXF];
#pragma unroll
    for (int x = 0; x < PXF; ++x) {
        const int prow = b_row0 + 32 * x;
        const int32_t p = m0 + prow;
        p_valid[x] = p < a.M;
        const int32_t pp = p_valid[x] ? p : 0;
        const int32_t rr = fdiv(pp, a.div_bw);
        const int32_t bx = pp - rr * a.bw;
        const int32_t n = fdiv(rr, a.div_bh);
        const int32_t by = rr - n * a.bh;
        dst[x] = a.out + (int64_t)n * a.out_sn + (int64_t)(a.y0 + by) * a.out_sh + (int64_t)(a.x0 + bx) * a.out_sw + oc0 * a.out_sc;
        a_corr[x] = a.dw != 0 ? a.dw * (sAsum[prow] + a.ktot * a.da) : 0;
    }
    if (a.dw != 0) epi_store<2, PXF, true>(a, es, acc, 0, noc, half, dst, p_valid, a_corr, mode, pu);
    else epi_store<2, PXF, false>(a, es, acc, 0, noc, half, dst, p_valid, a_corr, mode, pu);
}

}  // namespace

hipError_t launch_conv_gather(const ConvArgs& a, hipStream_t stream) {
    const unsigned gy = (unsigned)((a.bc + BN - 1) / BN);
    // Tile 256 pixels per workgroup only when that still leaves at least two workgroups per CU.
    const int64_t wg256 = (((int64_t)a.M + 255) / 256) * gy;
    if (wg256 >= 512) {
        const int64_t gx = ((int64_t)a.M + 255) / 256;
        if (gx > 0x7fffffffLL) return hipErrorInvalidValue;
        return emit(conv_igemm_kernel<2>, dim3(xcd_grid((unsigned)gx), gy), dim3(NTHREADS), 0, stream, a);
    } else {
        const int64_t gx = ((int64_t)a.M + 127) / 128;
        return emit(conv_igemm_kernel<1>, dim3(xcd_grid((unsigned)gx), gy), dim3(NTHREADS), 0, stream, a);
    }
}

// Launch arguments of a convolution over one box; hipSuccess, or the error to return.
static hipError_t make_conv_args(const TaskDev& t, const Box& box, ConvArgs& a) {
    a.in = t.in.data;
    a.in_sn = t.in.sn;
    a.in_sh = t.in.sh;
    a.in_sw = t.in.sw;
    a.H = t.in.h;
    a.W = t.in.w;
    a.IC = t.in.c;
    a.w = t.weights;
    a.w_soc = t.w_stride_oc;
    a.table = t.table;
    a.table_stride = t.table_stride;
    a.out = t.out.data;
    a.out_sn = t.out.sn;
    a.out_sh = t.out.sh;
    a.out_sw = t.out.sw;
    a.out_sc = t.out.sc;
    a.x0 = box.x0;
    a.y0 = box.y0;
    a.z0 = box.z0;
    a.bw = box.bw;
    a.bh = box.bh;
    a.bc = box.bc;
    const int64_t m64 = (int64_t)t.out.n * box.bh * box.bw;
    if (m64 >= 0x7fffffffLL) return hipErrorInvalidValue;
    a.M = (int32_t)m64;
    a.div_bw = make_fastdiv((uint32_t)box.bw);
    a.div_bh = make_fastdiv((uint32_t)box.bh);
    a.div_pitch = make_fastdiv(1);
    a.div_rows_full = make_fastdiv(1);
    a.KY = t.ky;
    a.KX = t.kx;
    a.SY = t.sy;
    a.SX = t.sx;
    a.PT = t.pt;
    a.PL = t.pl;
    a.ICG = t.in.c / 16;
    a.KG = t.ky * t.kx * a.ICG;
    a.ktot = t.ky * t.kx * t.in.c;
    const int32_t off_a = t.in.is_signed ? 0 : 128;
    const int32_t off_w = t.w_is_signed ? 0 : 128;
    a.a_xor = t.in.is_signed ? 0u : 0x80808080u;
    a.w_xor = t.w_is_signed ? 0u : 0x80808080u;
    a.da = off_a - t.in.zp;
    a.dw = off_w - t.w_zp;
    const uint32_t fb = (uint32_t)((t.in.zp - off_a) & 0xFF);
    a.fill = fb * 0x01010101u;
    a.fill_raw = (uint32_t)(t.in.zp & 0xFF);
    a.pitchpx = t.in.w + t.pl + t.pr;
    a.nslots_max = a.rows_max = a.nchunks = a.halo_bytes = 0;
    a.ppe = t.ppe;
    return hipSuccess;
}

static bool same_dense_tensor(const TensorDev& x, const TensorDev& y) {
    return x.data == y.data && x.n == y.n && x.h == y.h && x.w == y.w && x.c == y.c && x.sc == 1 && y.sc == 1 && x.sw == y.sw &&
           x.sh == y.sh && x.sn == y.sn && x.sw == x.c && x.sh == (int64_t)x.w * x.c && x.sn == (int64_t)x.h * x.sh;
}
static bool same_shape_dense(const TensorDev& x, const TensorDev& like) {
    return x.n == like.n && x.h == like.h && x.w == like.w && x.c == like.c && x.sc == 1 && x.sw == x.c &&
           x.sh == (int64_t)x.w * x.c && x.sn == (int64_t)x.h * x.sh;
}
static bool overlaps(const TensorDev& x, const TensorDev& y) {
    const uint8_t* xe = x.data + (int64_t)x.n * x.sn;
    const uint8_t* ye = y.data + (int64_t)y.n * y.sn;
    return x.data < ye && y.data < xe;
}

// Which convolutions take the LDS-tiled kernel: 0 = none of its shapes, else the shape (0 within a forced value: automatic).
static int tiled_shape_for(const ConvArgs& a) {
    if (tls_launch.per_xcd) return 0;
    const int forced = options().tiled;
    if (forced >= 0) return forced;
    // Fitted to a sweep of the ResNet-50 layer shapes at batch 32, 64, 128 and 256 (each layer alone, every kernel forced)
    // and to the whole graph at those batches. The 128 x 128 tile with steps of 128 bytes of the reduction (one barrier and
    // one LDS round trip per 32 matrix instructions of a wave; input channels a multiple of 128) is 3-25 % ahead of the
    // weights-resident kernels - 45 % for 3x3 over 512 channels - where the reduction is long and the output channels are
    // many. Inside the graph a launch of it costs ~1.5 us more than alone (the layer-alone sweep repeats one kernel, whose
    // weights then stay in L2 and whose launches overlap their own tails), so grids whose gain alone is 1-2 us are left to
    // the weights-resident kernels: from 1024 bytes of reduction it takes 384 workgroups (196 from 4096 bytes), from 512
    // bytes 512 workgroups of at least 256 channels - but not 256..511 channels over more than 1024 workgroups, where the
    // weights-resident kernels amortise their staging over many tiles per workgroup and win again. Shorter reductions and
    // fewer than 128 channels always lose. The 64-byte-step shape (input channels not a multiple of 128) is 9 % slower and
    // keeps the narrower window it was measured in. (The sweep ran the 128-byte steps with four waves per workgroup; the same
    // tile with eight waves - shape 6, what is returned now - is 1-3 % ahead of it on every layer of the window.)
    const int64_t k = (int64_t)a.KY * a.KX * a.IC;
    if (a.IC % 64 != 0 || a.dw != 0 || k < 512 || a.bc < 128) return 0;
    const int64_t groups = (((int64_t)a.M + 127) / 128) * ((a.bc + 127) / 128);
    if (a.IC % 128 != 0) return k >= 1024 && a.bc >= 256 && groups >= 384 && groups <= 1024 ? 1 : 0;
    bool use;
    if (k >= 1024) use = groups >= (k >= 4096 ? 196 : 384);
    else use = a.bc >= 256 && groups >= 512 && (a.bc >= 512 || groups <= 1024);
    return use ? 6 : 0;
}

// Which convolutions take the patch kernel (both operands in LDS, every input byte fetched once per workgroup).
static bool patch_wanted(const ConvArgs& a) {
    if (tls_launch.per_xcd) return false;
    const int forced = options().patch;
    if (forced >= 0) return forced != 0;
    // Measured against the weights-resident kernels over the ResNet-50 shapes at batch 32 .. 256 (each layer alone): ahead
    // by 6-17 % for 3x3 kernels at stride 1 over 64 input channels from about 100,000 output pixels and over 128 input
    // channels from about 50,000 (64 output channels per slice, sixteen waves); level or behind for everything else - 1x1
    // kernels (nothing to reuse), 256 and more input channels (a slice of 32 channels reads 0.75 KiB of LDS per matrix
    // instruction) and small layers (too few patches for the CUs).
    if (a.KY * a.KX < 2 || a.SY != 1 || a.SX != 1 || a.dw != 0 || a.bc < 64) return false;
    if (a.IC == 64) return a.M >= 100000;
    if (a.IC == 128) return a.M >= 50000;
    return false;
}

hipError_t launch_conv_fused_add(const TaskDev& conv, const Box& cb, const TaskDev& add, const Box& ab, hipStream_t stream) {
    if (options().no_fuse || (options().env_path && !tls_launch.per_xcd)) return hipErrorNotSupported;
    const TensorDev& o = conv.out;
    const bool conv_full = cb.x0 == 0 && cb.y0 == 0 && cb.z0 == 0 && cb.bw == o.w && cb.bh == o.h && cb.bc == o.c;
    const bool add_full = ab.x0 == 0 && ab.y0 == 0 && ab.z0 == 0 && ab.bw == add.out.w && ab.bh == add.out.h && ab.bc == add.out.c;
    if (!conv_full || !add_full || add.table != nullptr) return hipErrorNotSupported;
    const bool is_in1 = same_dense_tensor(add.in, o), is_in2 = same_dense_tensor(add.in2, o);
    if (is_in1 == is_in2) return hipErrorNotSupported;  // neither input, or both
    const TensorDev& other = is_in1 ? add.in2 : add.in;
    // The add must see the convolution's stored type; its other input and its output have the same dense shape and
    // do not touch the convolution's output (the output may be the other input: each element is read before it is written,
    // by the same lane).
    if ((is_in1 ? add.in : add.in2).is_signed != o.is_signed) return hipErrorNotSupported;
    if (!same_shape_dense(other, o) || !same_shape_dense(add.out, o) || overlaps(other, o) || overlaps(add.out, o)) return hipErrorNotSupported;
    if (overlaps(add.out, other) && add.out.data != other.data) return hipErrorNotSupported;
    // ... nor the convolution's operands
    if (overlaps(add.out, conv.in)) return hipErrorNotSupported;
    const uint8_t* const ob = add.out.data;
    const uint8_t* const oe = ob + (int64_t)add.out.n * add.out.sn;
    const uint8_t* const wb = conv.weights;
    const uint8_t* const we = wb + (int64_t)o.c * conv.w_stride_oc;
    const uint8_t* const tb = reinterpret_cast<const uint8_t*>(conv.table);
    const uint8_t* const te = tb + (int64_t)o.c * conv.table_stride * 4;
    if ((ob < we && wb < oe) || (ob < te && tb < oe)) return hipErrorNotSupported;
    FuseAdd fz;
    if (!eltwise_fuse_params(add, is_in1, &fz)) return hipErrorNotSupported;
    fz.other = other.data;
    fz.out = add.out.data;
    ConvArgs a;
    if (const hipError_t e = make_conv_args(conv, cb, a); e != hipSuccess) return e;
    if (a.M == 0 || cb.bc == 0) return hipErrorNotSupported;
    if (const int shape = tiled_shape_for(a)) {
        const hipError_t e = launch_conv_tiled(a, stream, shape, &fz);
        if (e != hipErrorNotSupported) return e;
    }
    return launch_conv_wres(a, stream, false, &fz);
}

hipError_t launch_conv(const TaskDev& t, const Box& box, hipStream_t stream) {
    ConvArgs a;
    if (const hipError_t e0 = make_conv_args(t, box, a); e0 != hipSuccess) return e0;
    if (a.M == 0 || box.bc == 0) return hipSuccess;
    if (tls_launch.per_xcd) return launch_conv_wres(a, stream, false);  // (nothing else takes part in persistent segments)
    // tuning and test knob: 1 = skip the weights-resident kernel, 2 = gather kernel only
    const int path = options().conv_path;
    // Reductions too long for one LDS slice: the halo kernel is the faster one for 3-wide kernels (measured on
    // 3x3 over 1024 channels), the chunked weights-resident kernel for everything else and for what the halo
    // kernel rejects.
    hipError_t e = hipErrorNotSupported;
    if (path == 0 && patch_wanted(a))
        e = launch_conv_patch(a, stream, options().patch >= 0 ? options().patch_nf : 4, options().patch_pr, options().patch >= 0 ? options().patch_waves : 16,
                              options().patch >= 0 ? options().patch_npx : 0);
    if (e != hipErrorNotSupported) return e;
    if (const int shape = path == 0 ? tiled_shape_for(a) : 0) e = launch_conv_tiled(a, stream, shape);
    if (e != hipErrorNotSupported) return e;
    e = path == 0 ? launch_conv_wres(a, stream, a.KX != 3) : hipErrorNotSupported;
    if (e != hipErrorNotSupported) return e;
    e = path <= 1 ? launch_conv_halo(a, stream) : hipErrorNotSupported;
    if (e != hipErrorNotSupported) return e;
    e = path == 0 && a.KX == 3 ? launch_conv_wres(a, stream, true) : hipErrorNotSupported;
    if (e != hipErrorNotSupported) return e;
    return launch_conv_gather(a, stream);
}

}  // namespace nce
