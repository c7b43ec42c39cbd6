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
#include <numeric>
#include <cstdlib>

namespace nce {
namespace {

constexpr int JMAX = 8;  // halo 16-byte loads per thread per input slice

template <int WN, int WP, int AF, int BF, int KX>
__global__ __launch_bounds__(64 * WN * WP) void conv_halo_kernel(ConvArgs a) {
    prefetch_kernel_arguments<sizeof(ConvArgs)>();
    constexpr int NT = 64 * WN * WP;
    constexpr int BN = WN * AF * 32;
    constexpr int BM = WP * BF * 32;
    constexpr int WCH = BN * KX * 4;         // 16-byte weight chunks per step
    constexpr int WI = (WCH + NT - 1) / NT;  // ... per thread
    constexpr int WBYTES = BN * KX * 64;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sHalo = smem;
    uint8_t* sWt = smem + a.halo_bytes;
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

    const uint32_t ntiles = ((uint32_t)a.M + BM - 1) / BM;
    const uint32_t tile = xcd_tile(blockIdx.x, ntiles);
    if (tile >= ntiles) return;  // uniform for the whole workgroup

    epi_load_table(a, es, tid, NT, BN, oc0, noc);
    __syncthreads();  // the zeroed weight sums are in place before any wave adds to them (store_weights below)

    // ---- tile geometry (uniform) ------------------------------------------------------------
    const int32_t m0 = tile * BM;
    const int32_t m_end = min(m0 + BM, a.M);
    const int32_t rr_first = fdiv(m0, a.div_bw);  // box rows are numbered n * bh + by
    const int32_t rr_last = fdiv(m_end - 1, a.div_bw);
    const int32_t n_first = fdiv(rr_first, a.div_bh);
    const int by_first = rr_first - n_first * a.bh;
    const int rows0 = (a.bh - 1 - by_first) * a.SY + a.KY;  // slots of the first image if it runs to its end
    const int rows_full = (a.bh - 1) * a.SY + a.KY;        // slots of a whole image

    auto first_slot_of = [&](int32_t rr) {
        const int32_t n = fdiv(rr, a.div_bh);
        const int by = rr - n * a.bh;
        const int seg = n - n_first;
        return seg == 0 ? (by - by_first) * a.SY : rows0 + (seg - 1) * rows_full + by * a.SY;
    };
    const int nslots = first_slot_of(rr_last) + a.KY;
    const int total_h = nslots * a.pitchpx * 4;

    // ---- staging assignment -------------------------------------------------------------------
    const uint8_t* h_src[JMAX];  // nullptr: fill
    int32_t h_dst[JMAX];         // -1: nothing to stage
#pragma unroll
    for (int j = 0; j < JMAX; ++j) {
        const int h = tid + NT * j;
        h_src[j] = nullptr;
        h_dst[j] = -1;
        if (h < total_h) {
            const int pxl = h >> 2;
            const int slot = fdiv(pxl, a.div_pitch);
            const int ix = pxl - slot * a.pitchpx - a.PL;
            int seg = 0, iy = (a.y0 + by_first) * a.SY - a.PT + slot;
            if (slot >= rows0) {
                const int q = slot - rows0;
                const int sq = fdiv(q, a.div_rows_full);
                seg = 1 + sq;
                iy = a.y0 * a.SY - a.PT + (q - sq * rows_full);
            }
            h_dst[j] = pxl * 64 + (((h & 3) ^ ((pxl >> 2) & 3)) << 4);
            if (iy >= 0 && iy < a.H && ix >= 0 && ix < a.W)
                h_src[j] = a.in + (int64_t)(n_first + seg) * a.in_sn + (int64_t)iy * a.in_sh + (int64_t)ix * a.in_sw + ((h & 3) << 4);
        }
    }
    const uint8_t* w_src[WI];  // nullptr: zero (channel beyond the box)
    int32_t w_dst[WI];
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const int q = tid + NT * i;
        w_src[i] = nullptr;
        w_dst[i] = -1;
        if (q < WCH) {
            const int row = q / (KX * 4);
            const int kx = (q - row * (KX * 4)) >> 2;
            const int lrow = (row & ~31) | row_of_chan(row & 31);
            w_dst[i] = (kx * BN + lrow) * 64 + (((q & 3) ^ ((lrow >> 2) & 3)) << 4);
            if (row < noc) w_src[i] = a.w + (int64_t)(oc0 + row) * a.w_soc + (int64_t)kx * a.IC + ((q & 3) << 4);
        }
    }
    const int grp16 = (tid & 3) << 4;  // both staging lists give a thread the same 16-byte column (NT % 4 == 0)

    const uint4 fill4 = make_uint4(a.fill, a.fill, a.fill, a.fill);
    const int nsteps = a.nchunks * a.KY;
    // step index -> (64-channel slice, kernel row)
    auto load_weights = [&](uint4 (&rw)[WI], int step) {
        const int c = step / a.KY, ky = step - c * a.KY;
        const int64_t koff = (int64_t)ky * KX * a.IC + c * 64;
        const bool col_ok = c * 64 + grp16 < a.IC;
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (w_src[i] != nullptr && col_ok && step < nsteps) {
                v = *reinterpret_cast<const uint4*>(w_src[i] + koff);
                v.x ^= a.w_xor;
                v.y ^= a.w_xor;
                v.z ^= a.w_xor;
                v.w ^= a.w_xor;
            }
            rw[i] = v;
        }
    };
    auto store_weights = [&](const uint4 (&rw)[WI], int buf) {
#pragma unroll
        for (int i = 0; i < WI; ++i)
            if (w_dst[i] >= 0) {
                *reinterpret_cast<uint4*>(sWt + buf * WBYTES + w_dst[i]) = rw[i];
                if (a.da != 0) atomicAdd(&sWsum[(tid + NT * i) / (KX * 4)], bytesum(rw[i]));
            }
    };
    uint4 rh[JMAX];
    auto load_halo = [&](int c) {
        const bool col_ok = c * 64 + grp16 < a.IC;
#pragma unroll
        for (int j = 0; j < JMAX; ++j) {
            uint4 v = fill4;
            if (h_src[j] != nullptr && col_ok) {
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

    // Everything the first step needs is requested before anything is waited for.
    uint4 rw[WI];
    load_weights(rw, 0);
    load_halo(0);

    // ---- MFMA operand addressing --------------------------------------------------------------
    int32_t b_px[BF];  // LDS pixel index of tap (0, 0) for this lane's pixel of fragment x
    int32_t b_rr[BF];  // box row and column of that pixel
    int32_t b_bx[BF];
    bool valid[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        const int32_t p = m0 + (wp * BF + x) * 32 + l32;
        valid[x] = p < m_end;
        const int32_t pc = valid[x] ? p : m_end - 1;  // lanes past the end compute a duplicate
        b_rr[x] = fdiv(pc, a.div_bw);
        b_bx[x] = pc - b_rr[x] * a.bw;
        b_px[x] = first_slot_of(b_rr[x]) * a.pitchpx + (a.x0 + b_bx[x]) * a.SX;
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

    store_weights(rw, 0);
    store_halo();
    __syncthreads();

    // ---- main loop: one step = one kernel row (KX taps) of one 64-channel slice ----------------
    // The weights of the next step and (on the last kernel row) the halo of the next slice are
    // requested before this step's MFMAs and written to LDS after them.
    int c = 0, ky = 0;
    for (int s = 0; s < nsteps; ++s) {
        const bool last_row = ky == a.KY - 1;
        const bool new_halo = last_row && c + 1 < a.nchunks;
        load_weights(rw, s + 1);
        if (new_halo) load_halo(c + 1);

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
        if (s + 1 < nsteps) store_weights(rw, (s + 1) & 1);
        if (new_halo) {
            __syncthreads();  // every wave is done with the current slice
            store_halo();
        }
        __syncthreads();
        if (last_row) {
            ky = 0;
            ++c;
        } else {
            ++ky;
        }
    }

    // ---- PPE + store --------------------------------------------------------------------------
    PpeF64 pu;
    const int mode = epi_constants(a, es, tid, NT, BN, &pu);
    uint8_t* dst[BF];
    int32_t acorr[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        const int32_t n = fdiv(b_rr[x], a.div_bh);
        const int by = b_rr[x] - n * a.bh;
        dst[x] = a.out + (int64_t)n * a.out_sn + (int64_t)(a.y0 + by) * a.out_sh + (int64_t)(a.x0 + b_bx[x]) * a.out_sw + oc0 * a.out_sc;
        acorr[x] = 0;
    }
    epi_store<AF, BF, false>(a, es, acc, wn * AF * 32, noc, half, dst, valid, acorr, mode, pu);
}

// Exact staging bounds of a tiling: the largest number of output rows and of input-row slots any
// tile of bm pixels touches (same arithmetic as the kernel).
void tile_bounds(const ConvArgs& a, int bm, int* rows_max, int* nslots_max) {
    int rmax = 0, smax = 0;
    const int64_t ntiles = ((int64_t)a.M + bm - 1) / bm;
    const int rows_full = (a.bh - 1) * a.SY + a.KY;
    // A tile's extent depends only on where in an image it starts, and the start positions repeat after
    // bw * bh / gcd(bm, bw * bh) tiles (a clipped last tile touches no more than the full tile of its position): the walk
    // is bounded by the image, not by the batch.
    const int64_t img = (int64_t)a.bw * a.bh;
    const int64_t walk = std::min(ntiles, img / std::gcd<int64_t>(bm, img) + 1);
    for (int64_t t = 0; t < walk; ++t) {
        const int64_t m0 = t * bm, m_end = std::min<int64_t>(m0 + bm, (int64_t)a.M);
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
    const size_t lds = (size_t)a.halo_bytes + 2 * (size_t)BN * KX * 64;
    *fits = lds <= 140 * 1024;
    if (!*fits) return hipSuccess;
    const int64_t gx = ((int64_t)a.M + BM - 1) / BM;
    const unsigned gy = (unsigned)((a.bc + BN - 1) / BN);
    if (gx > 0x7fffffffLL) return hipErrorInvalidValue;
    auto kernel = &conv_halo_kernel<WN, WP, AF, BF, KX>;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    return emit(kernel, dim3(xcd_grid((unsigned)gx), gy), dim3(NT), lds, stream, a);
}

// Tile shapes: {channel waves, pixel waves, channel fragments, pixel fragments per wave}.
//   0: 128 ch x 256 px, 4 waves   1: 64 ch x 256 px, 4 waves   2: 64 ch x 128 px, 4 waves   3: 64 ch x 64 px, 2 waves
template <int KX>
hipError_t launch_tile(int tile, const ConvArgs& a, hipStream_t stream, bool* fits) {
    switch (tile) {
    case 0: return try_launch<2, 2, 2, 4, KX>(a, stream, fits);
    case 1: return try_launch<1, 4, 2, 2, KX>(a, stream, fits);
    case 2: return try_launch<1, 4, 2, 1, KX>(a, stream, fits);
    default: return try_launch<1, 2, 2, 1, KX>(a, stream, fits);
    }
}

template <int KX>
hipError_t launch_kx(const ConvArgs& a, hipStream_t stream) {
    // Big tiles pay off only with a long reduction (their epilogue and staging run at one wave per
    // SIMD); short reductions and small problems take small tiles for occupancy and CU coverage.
    const int64_t px256 = (a.M + 255) / 256, px128 = (a.M + 127) / 128;
    const int64_t ch128 = (a.bc + 127) / 128, ch64 = (a.bc + 63) / 64;
    // Measured on MI355X: 64 ch x 128 px is the best all-round shape; 1x1 kernels with enough
    // workgroups prefer 64 ch x 256 px. The 128-channel tile (one wave per SIMD) never wins.
    int first = 2;
    if (KX == 1 && px256 * ch64 >= 384) first = 1;
    (void)px128;
    (void)ch128;
    const int forced = options().halo_tile;  // tuning knob: force one tile shape (0..3)
    if (forced >= 0 && forced <= 3) first = forced;
    for (int tile = first; tile <= 3; ++tile) {
        bool fits = false;
        const hipError_t e = launch_tile<KX>(tile, a, stream, &fits);
        if (fits || e != hipSuccess) return e;
    }
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_conv_halo(const ConvArgs& a_in, hipStream_t stream) {
    if (a_in.dw != 0 || a_in.IC < 64) return hipErrorNotSupported;
    ConvArgs a = a_in;
    a.nchunks = (a.IC + 63) / 64;
    a.div_pitch = make_fastdiv((uint32_t)a.pitchpx);
    a.div_rows_full = make_fastdiv((uint32_t)((a.bh - 1) * a.SY + a.KY));
    if (a.KX == 1) return launch_kx<1>(a, stream);
    if (a.KX == 3) return launch_kx<3>(a, stream);
    return hipErrorNotSupported;
}

}  // namespace nce
