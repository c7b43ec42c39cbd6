// CONV task, halo-staged implicit GEMM for 1x1 / 3-wide kernels with at least 64 input channels.
//
// A workgroup owns BM consecutive output pixels (linear over batch, row, column) x BN output channels.
// Per 64-channel slice of the input it stages ONCE, in LDS, every input row those pixels need
// ("slots": consecutive input rows per image, each padded left/right with the zero-point fill), so the
// KY*KX taps of the kernel all read the same staged bytes at a per-tap uniform offset:
//     LDS pixel(lane, ky, kx) = base(lane) + ky * pitch + kx
// instead of re-fetching the activations from L2 once per tap. Weights stream through a double-buffered
// LDS tile of one kernel row (KX taps x BN channels x 64 bytes) per step. Both LDS tiles use a 64-byte
// pitch with the 16-byte column XOR-swizzled by (row >> 2) & 3, which makes the 128-bit MFMA operand
// reads of 16 consecutive rows hit 16 different bank groups.
//
// Global loads of the next step (weights) and the next slice (halo) are issued before the MFMAs of the
// current step and written to LDS after them, so their latency hides behind a whole kernel row of
// matrix instructions. Semantics and the fused PPE are the ones of nce_conv.hip.
#include "nce_conv_common.h"

#include <algorithm>

namespace nce {
namespace {

constexpr int JMAX = 8;  // halo 16-byte loads per thread per input slice

template <int WN, int WP, int AF, int BF, int KX>
__global__ __launch_bounds__(64 * WN * WP) void conv_halo_kernel(ConvArgs a) {
    constexpr int NT = 64 * WN * WP;
    constexpr int BN = WN * AF * 32;
    constexpr int BM = WP * BF * 32;
    constexpr int WCH = BN * KX * 4;         // 16-byte weight chunks per step
    constexpr int WI = (WCH + NT - 1) / NT;  // ... per thread
    constexpr int WBYTES = BN * KX * 64;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sHalo = smem;
    uint8_t* sWt = smem + a.halo_bytes;
    int64_t* sSlotOff = reinterpret_cast<int64_t*>(sWt + 2 * WBYTES);
    int32_t* sFirst = reinterpret_cast<int32_t*>(sSlotOff + a.nslots_max);
    __shared__ int32_t sW2[BN], sBias[BN], sWsum[BN], sCorr[BN];
    __shared__ double sM[BN], sBc[BN];
    const EpiSmem es = {sM, sBc, sW2, sBias, sCorr, sWsum};

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave % WN;  // position along channels
    const int wp = wave / WN;  // position along pixels
    const int half = lane >> 5;
    const int l32 = lane & 31;

    const int32_t oc0 = a.z0 + blockIdx.y * BN;
    const int32_t noc = min(BN, a.z0 + a.bc - oc0);

    // ---- tile geometry (uniform) ------------------------------------------------------------
    const int64_t m0 = (int64_t)blockIdx.x * BM;
    const int64_t m_end = min(m0 + (int64_t)BM, a.M);
    const int64_t rr_first = m0 / a.bw;  // box rows are numbered n * bh + by
    const int64_t rr_last = (m_end - 1) / a.bw;
    const int rows_out = (int)(rr_last - rr_first + 1);
    const int64_t n_first = rr_first / a.bh;
    const int by_first = (int)(rr_first - n_first * a.bh);
    const int rows0 = (a.bh - 1 - by_first) * a.SY + a.KY;  // slots of the first image if it runs to its end
    const int rows_full = (a.bh - 1) * a.SY + a.KY;        // slots of a whole image

    auto first_slot_of = [&](int64_t rr) {
        const int64_t n = rr / a.bh;
        const int by = (int)(rr - n * a.bh);
        const int seg = (int)(n - n_first);
        return seg == 0 ? (by - by_first) * a.SY : rows0 + (seg - 1) * rows_full + by * a.SY;
    };
    const int nslots = first_slot_of(rr_last) + a.KY;
    const int total_h = nslots * a.pitchpx * 4;

    epi_load_table(a, es, tid, NT, BN, oc0, noc);
    for (int r = tid; r < rows_out; r += NT) sFirst[r] = first_slot_of(rr_first + r);
    for (int s = tid; s < nslots; s += NT) {
        int seg, iy;
        if (s < rows0) {
            seg = 0;
            iy = (a.y0 + by_first) * a.SY - a.PT + s;
        } else {
            const int q = s - rows0;
            seg = 1 + q / rows_full;
            iy = a.y0 * a.SY - a.PT + (q - (seg - 1) * rows_full);
        }
        const int64_t n = n_first + seg;
        sSlotOff[s] = (iy >= 0 && iy < a.H) ? n * a.in_sn + (int64_t)iy * a.in_sh : (int64_t)-1;
    }
    __syncthreads();

    // ---- staging assignment -------------------------------------------------------------------
    const uint8_t* h_src[JMAX];  // nullptr: fill
    int32_t h_dst[JMAX];         // -1: nothing to stage
    int32_t h_grp[JMAX];
#pragma unroll
    for (int j = 0; j < JMAX; ++j) {
        const int h = tid + NT * j;
        h_src[j] = nullptr;
        h_dst[j] = -1;
        h_grp[j] = h & 3;
        if (h < total_h) {
            const int pxl = h >> 2;
            const int slot = pxl / a.pitchpx;
            const int ix = pxl - slot * a.pitchpx - a.PL;
            const int64_t off = sSlotOff[slot];
            h_dst[j] = pxl * 64 + (((h & 3) ^ ((pxl >> 2) & 3)) << 4);
            if (off >= 0 && ix >= 0 && ix < a.W) h_src[j] = a.in + off + (int64_t)ix * a.in_sw + ((h & 3) << 4);
        }
    }
    const uint8_t* w_src[WI];  // nullptr: zero (channel beyond the box)
    int32_t w_dst[WI];
    int32_t w_row[WI];
    int32_t w_grp[WI];
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const int q = tid + NT * i;
        w_src[i] = nullptr;
        w_dst[i] = -1;
        w_row[i] = 0;
        w_grp[i] = q & 3;
        if (q < WCH) {
            const int row = q / (KX * 4);
            const int kx = (q - row * (KX * 4)) >> 2;
            const int lrow = (row & ~31) | row_of_chan(row & 31);
            w_row[i] = row;
            w_dst[i] = (kx * BN + lrow) * 64 + (((q & 3) ^ ((lrow >> 2) & 3)) << 4);
            if (row < noc) w_src[i] = a.w + (int64_t)(oc0 + row) * a.w_soc + (int64_t)kx * a.IC + ((q & 3) << 4);
        }
    }

    uint4 rw[WI], rh[JMAX];
    const uint4 fill4 = make_uint4(a.fill, a.fill, a.fill, a.fill);
    auto load_weights = [&](int c, int ky) {
        const int64_t koff = (int64_t)ky * KX * a.IC + c * 64;
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (w_src[i] != nullptr && c * 64 + (w_grp[i] << 4) < a.IC) {
                v = *reinterpret_cast<const uint4*>(w_src[i] + koff);
                v.x ^= a.w_xor;
                v.y ^= a.w_xor;
                v.z ^= a.w_xor;
                v.w ^= a.w_xor;
                if (a.da != 0) atomicAdd(&sWsum[w_row[i]], bytesum(v));
            }
            rw[i] = v;
        }
    };
    auto store_weights = [&](int buf) {
#pragma unroll
        for (int i = 0; i < WI; ++i)
            if (w_dst[i] >= 0) *reinterpret_cast<uint4*>(sWt + buf * WBYTES + w_dst[i]) = rw[i];
    };
    auto load_halo = [&](int c) {
#pragma unroll
        for (int j = 0; j < JMAX; ++j) {
            uint4 v = fill4;
            if (h_src[j] != nullptr && c * 64 + (h_grp[j] << 4) < a.IC) {
                v = *reinterpret_cast<const uint4*>(h_src[j] + c * 64);
                v.x ^= a.a_xor;
                v.y ^= a.a_xor;
                v.z ^= a.a_xor;
                v.w ^= a.a_xor;
            }
            rh[j] = v;
        }
    };
    auto store_halo = [&]() {
#pragma unroll
        for (int j = 0; j < JMAX; ++j)
            if (h_dst[j] >= 0) *reinterpret_cast<uint4*>(sHalo + h_dst[j]) = rh[j];
    };

    // ---- MFMA operand addressing --------------------------------------------------------------
    int32_t b_px[BF];      // LDS pixel index of tap (0, 0) for this lane's pixel of fragment x
    int64_t b_p[BF];       // linear output pixel
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        const int64_t p = m0 + (wp * BF + x) * 32 + l32;
        b_p[x] = p;
        const int64_t pc = p < m_end ? p : m_end - 1;  // lanes past the end compute a duplicate
        const int64_t rr = pc / a.bw;
        const int bx = (int)(pc - rr * a.bw);
        b_px[x] = sFirst[(int)(rr - rr_first)] * a.pitchpx + (a.x0 + bx) * a.SX;
    }
    int32_t a_row[AF];
#pragma unroll
    for (int f = 0; f < AF; ++f) a_row[f] = (wn * AF + f) * 32 + l32;

    v16i acc[AF][BF];
#pragma unroll
    for (int f = 0; f < AF; ++f)
#pragma unroll
        for (int x = 0; x < BF; ++x)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[f][x][v] = 0;

    // ---- main loop: one step = one kernel row (KX taps) of one 64-channel slice --------------
    const int nsteps = a.nchunks * a.KY;
    load_weights(0, 0);
    load_halo(0);
    store_weights(0);
    store_halo();
    __syncthreads();
    int c = 0, ky = 0;
    for (int s = 0; s < nsteps; ++s) {
        int c2 = c, ky2 = ky + 1;
        if (ky2 == a.KY) {
            ky2 = 0;
            ++c2;
        }
        const bool more = s + 1 < nsteps;
        const bool new_halo = more && ky2 == 0;
        if (more) load_weights(c2, ky2);
        if (new_halo) load_halo(c2);

        const uint8_t* wt = sWt + (s & 1) * WBYTES;
#pragma unroll
        for (int kx = 0; kx < KX; ++kx) {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const int chunk = kk * 2 + half;
                v4i fa[AF], fb[BF];
#pragma unroll
                for (int f = 0; f < AF; ++f)
                    fa[f] = *reinterpret_cast<const v4i*>(wt + (kx * BN + a_row[f]) * 64 + ((chunk ^ ((a_row[f] >> 2) & 3)) << 4));
#pragma unroll
                for (int x = 0; x < BF; ++x) {
                    const int px = b_px[x] + ky * a.pitchpx + kx;
                    fb[x] = *reinterpret_cast<const v4i*>(sHalo + px * 64 + ((chunk ^ ((px >> 2) & 3)) << 4));
                }
#pragma unroll
                for (int f = 0; f < AF; ++f)
#pragma unroll
                    for (int x = 0; x < BF; ++x)
                        acc[f][x] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[f], fb[x], acc[f][x], 0, 0, 0);
            }
        }
        if (more) store_weights((s + 1) & 1);
        if (new_halo) {
            __syncthreads();  // every wave is done with the current slice
            store_halo();
        }
        __syncthreads();
        c = c2;
        ky = ky2;
    }

    // ---- PPE + store --------------------------------------------------------------------------
    PpeF64 pu;
    const int mode = epi_constants(a, es, tid, NT, BN, &pu);
    uint8_t* dst[BF];
    bool valid[BF];
    int32_t acorr[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        valid[x] = b_p[x] < m_end;
        const int64_t pc = valid[x] ? b_p[x] : m_end - 1;
        const int64_t rr = pc / a.bw;
        const int bx = (int)(pc - rr * a.bw);
        const int64_t n = rr / a.bh;
        const int by = (int)(rr - n * a.bh);
        dst[x] = a.out + n * a.out_sn + (int64_t)(a.y0 + by) * a.out_sh + (int64_t)(a.x0 + bx) * a.out_sw + oc0;
        acorr[x] = 0;
    }
    epi_store<AF, BF, false>(a, es, acc, wn * AF * 32, noc, half, dst, valid, acorr, mode, pu);
}

// Exact staging bounds of a tiling: the largest number of output rows and of input-row slots any
// tile of bm pixels touches (same arithmetic as the kernel).
void tile_bounds(const ConvArgs& a, int bm, int* rows_max, int* nslots_max) {
    int rmax = 0, smax = 0;
    const int64_t ntiles = (a.M + bm - 1) / bm;
    const int rows_full = (a.bh - 1) * a.SY + a.KY;
    for (int64_t t = 0; t < ntiles; ++t) {
        const int64_t m0 = t * bm, m_end = std::min<int64_t>(m0 + bm, a.M);
        const int64_t rr_first = m0 / a.bw, rr_last = (m_end - 1) / a.bw;
        const int64_t n_first = rr_first / a.bh, n_last = rr_last / a.bh;
        const int by_first = (int)(rr_first - n_first * a.bh), by_last = (int)(rr_last - n_last * a.bh);
        const int rows0 = (a.bh - 1 - by_first) * a.SY + a.KY;
        const int seg = (int)(n_last - n_first);
        const int first = seg == 0 ? (by_last - by_first) * a.SY : rows0 + (seg - 1) * rows_full + by_last * a.SY;
        rmax = std::max(rmax, (int)(rr_last - rr_first + 1));
        smax = std::max(smax, first + a.KY);
    }
    *rows_max = rmax;
    *nslots_max = smax;
}

template <int WN, int WP, int AF, int BF, int KX>
hipError_t try_launch(ConvArgs a, hipStream_t stream, bool* fits) {
    constexpr int NT = 64 * WN * WP;
    constexpr int BN = WN * AF * 32;
    constexpr int BM = WP * BF * 32;
    tile_bounds(a, BM, &a.rows_max, &a.nslots_max);
    const int64_t halo_px = (int64_t)a.nslots_max * a.pitchpx;
    *fits = halo_px * 4 <= (int64_t)JMAX * NT;
    if (!*fits) return hipSuccess;
    a.halo_bytes = (int32_t)(halo_px * 64);
    const size_t lds = (size_t)a.halo_bytes + 2 * (size_t)BN * KX * 64 + 8 * (size_t)a.nslots_max + 4 * (size_t)a.rows_max + 16;
    *fits = lds <= 140 * 1024;
    if (!*fits) return hipSuccess;
    const int64_t gx = (a.M + BM - 1) / BM;
    const unsigned gy = (unsigned)((a.bc + BN - 1) / BN);
    if (gx > 0x7fffffffLL) return hipErrorInvalidValue;
    auto kernel = &conv_halo_kernel<WN, WP, AF, BF, KX>;
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)gx, gy), dim3(NT), lds, stream, a);
    return hipGetLastError();
}

template <int KX>
hipError_t launch_kx(const ConvArgs& a, hipStream_t stream) {
    // Largest tile that still gives every CU a few workgroups; smaller tiles for small problems.
    const int64_t wg_big = ((a.M + 255) / 256) * ((a.bc + 127) / 128);
    const int64_t wg_mid = ((a.M + 255) / 256) * ((a.bc + 63) / 64);
    const int64_t wg_small = ((a.M + 127) / 128) * ((a.bc + 63) / 64);
    bool fits = false;
    hipError_t e;
    if (a.bc >= 128 && wg_big >= 512) {
        e = try_launch<2, 2, 2, 4, KX>(a, stream, &fits);
        if (fits || e != hipSuccess) return e;
    }
    if (wg_mid >= 512) {
        e = try_launch<1, 4, 2, 2, KX>(a, stream, &fits);
        if (fits || e != hipSuccess) return e;
    }
    if (wg_small >= 256) {
        e = try_launch<1, 4, 2, 1, KX>(a, stream, &fits);
        if (fits || e != hipSuccess) return e;
    }
    e = try_launch<1, 2, 2, 1, KX>(a, stream, &fits);
    if (fits || e != hipSuccess) return e;
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_conv_halo(const ConvArgs& a_in, hipStream_t stream) {
    if (a_in.dw != 0 || a_in.IC < 64) return hipErrorNotSupported;
    ConvArgs a = a_in;
    a.nchunks = (a.IC + 63) / 64;
    if (a.KX == 1) return launch_kx<1>(a, stream);
    if (a.KX == 3) return launch_kx<3>(a, stream);
    return hipErrorNotSupported;
}

}  // namespace nce
