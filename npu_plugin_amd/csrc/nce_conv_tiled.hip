// CONV task, LDS-tiled implicit GEMM on v_mfma_i32_16x16x64_i8 for layers with many output channels.
//
// A workgroup owns BM = 16*TM*WM output pixels x BN = 16*TN*WN output channels. Both operands of a reduction
// step (64 bytes of the OYXI weight rows; the same 64 input channels of one tap of every pixel) are staged in
// LDS once per workgroup and shared by its waves: the WN waves along the channels read the same activation
// rows, the WM waves along the pixels the same weight rows. Per step a wave reads TN + TM operand fragments
// for TN*TM matrix instructions (the weights-resident kernel, whose waves share nothing, reads its
// activations from global memory once per wave and tops out on the CU's L1 path).
//
// Staging: global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into LDS (no registers,
// no LDS store instruction): one instruction of a wave fills one 1 KiB block = 16 rows x 64 bytes, lane 4p + j
// at byte 16 * (4p + j) of the block. Which 16-byte piece of row p that lane FETCHES is the layout: piece
// j ^ swz(p), so that the row-per-lane operand reads spread over all banks while four neighbouring lanes still
// fetch one row's 64 contiguous bytes. NS stages of (BM + BN) * 64 bytes form a ring: the requests of step
// s + NS - 1 are issued when step s begins, so NS - 1 steps of loads are in flight per workgroup, and one
// barrier per step orders "my requests for this stage have landed" (s_waitcnt vmcnt) before every wave's reads.
// u8 operands are re-biased (x ^ 0x80) in registers after the operand read; taps outside the image fetch a
// line holding the input zero point. With an input zero point away from the storage offset the per-channel
// weight sums come out of the matrix unit (one more instruction per weight fragment and step, against ones).
//
// Conditions (checked on the host): input channels a multiple of 64, weights zero point equal to their
// storage offset, kernel up to 32 x 32. Semantics and the fused PPE are those of the weights-resident kernel
// (nce_conv_epi.h).
#include "nce_conv_epi.h"
#include "nce_conv_lds.h"

#include <algorithm>
#include <cstring>
#include <type_traits>

namespace nce {

namespace {

using namespace wres_detail;

struct TiledArgs {
    ConvArgs a;
    int32_t nsteps;   // 64-byte reduction steps: KY * KX * IC / 64
    int32_t nc64;     // 64-byte chunks along IC
    uint32_t ntm;     // pixel tiles
    uint32_t ntn;     // channel tiles
    int32_t inside;   // every tap of every pixel of the box lies inside the image
    int64_t row_adv;  // input offset from the last tap of a kernel row to the first of the next: in_sh - KX * in_sw
    FuseAdd fz;       // FZ kernels only
};

using namespace lds_detail;  // swz (bank-conflict-free piece placement), vmcnt_imm, gptr_t / lptr_t

// Waves per SIMD the register budget must allow (vector + accumulation registers share 512 per lane and SIMD): two
// workgroups of four waves, or one of eight, per CU at the least - a lone wave per SIMD leaves every LDS and barrier
// round trip of the step loop exposed. Eight waves of 32 x 64 outputs (eight accumulator fragments) fit 128 registers: two
// such workgroups share a CU, four waves per SIMD.
constexpr int tiled_min_waves(int nwaves, int frags) {
    return nwaves >= 8 && frags <= 8 ? 4 : 2;
}

template <int WM, int WN, int TM, int TN, int NS, int KC, bool FZ>
__global__ __launch_bounds__(64 * WM * WN, tiled_min_waves(WM * WN, TM * TN)) void conv_tiled_kernel(TiledArgs w) {
    prefetch_kernel_arguments<sizeof(TiledArgs)>();
    constexpr int NW = WM * WN;
    constexpr int BM = 16 * TM * WM;
    constexpr int BN = 16 * TN * WN;
    constexpr int CW = 16 * TN;              // channels per wave
    constexpr int ABLK = BN / 16;            // 1 KiB blocks of the weight tile
    constexpr int NA = ABLK / NW;            // blocks of the weight tile one wave fetches per step
    constexpr int NB = (BM / 16) / NW;       // blocks of the activation tile
    constexpr int CHUNK = (BM + BN) * 64;    // bytes of one 64-byte slice of the reduction: weight rows, then activation rows
    constexpr int STAGE = CHUNK * KC;        // bytes of one LDS stage: KC slices (a step covers 64 * KC bytes of the reduction)
    static_assert(TN == 2 || TN == 4, "channel fragments per wave");
    static_assert(ABLK % NW == 0 && (BM / 16) % NW == 0, "blocks divide among the waves");
    static_assert(!FZ || TN == 4, "fused add: a lane holds 16 channels");
    static_assert(NS >= 2 && (NS - 2) * (NA + NB) * KC < 64, "ring depth against the 6-bit load counter");
    const ConvArgs& a = w.a;

    extern __shared__ __attribute__((aligned(16))) uint8_t sT[];  // [stage][weights BN rows | activations BM rows] x 64 bytes
    __shared__ int64_t sOutOff[BM];   // output byte offset of the tile's pixels (channel 0 of the tensor)
    __shared__ int32_t sW2[BN], sBias[BN], sWsum[BN];
    __shared__ int32_t sCorr[BN];     // integer path: da * sum of weights; high-word path: scaled multiplier
    __shared__ double sM[BN], sBfull[BN];
    __shared__ int32_t sFlags;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % WN;  // position along channels
    const int wm = wave / WN;  // position along pixels
    const int c16 = lane & 15;

    const uint32_t ntotal = w.ntm * w.ntn;
    const uint32_t lid = xcd_tile(blockIdx.x, ntotal);
    if (lid >= ntotal) return;  // uniform for the whole workgroup
    const uint32_t mt = lid / w.ntn, nt = lid - mt * w.ntn;
    const int32_t oc0 = a.z0 + (int32_t)nt * BN;
    const int32_t noc = min(BN, a.z0 + a.bc - oc0);
    const int32_t m0 = (int32_t)mt * BM;

    // ---- what this thread fetches: row lane / 4 of the blocks wave, wave + NW, ... ; position lane % 4 -----------
    const int prow = lane >> 2;
    const int pj = (lane & 3) ^ swz(prow);  // the piece that belongs at this lane's position
    const uint8_t* wsrc[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int r = (wave + NW * i) * 16 + prow;  // row of the weight tile: fragment r / 16, wave group r / CW
        const int cl = (r / CW) * CW + channel_of_frag_row<TN>((r % CW) >> 4, r & 15);
        const int ch = min(cl, noc - 1);  // rows past the box's last channel duplicate it (their results are not stored)
        wsrc[i] = a.w + (int64_t)(oc0 + ch) * a.w_soc + pj * 16;
    }
    const uint8_t* bsrc[NB];
    uint32_t rows[NB], cols[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int r = (wave + NW * i) * 16 + prow;  // pixel of the tile
        const int32_t p = min(m0 + r, a.M - 1);     // pixels past the end duplicate the last one
        const int32_t rr = fdiv(p, a.div_bw);
        const int32_t bx = p - rr * a.bw;
        const int32_t n = fdiv(rr, a.div_bh);
        const int32_t by = rr - n * a.bh;
        const int32_t iy0 = (a.y0 + by) * a.SY - a.PT;
        const int32_t ix0 = (a.x0 + bx) * a.SX - a.PL;
        bsrc[i] = a.in + (int64_t)n * a.in_sn + (int64_t)iy0 * a.in_sh + (int64_t)ix0 * a.in_sw + pj * 16;
        rows[i] = bit_range(max(0, -iy0), min(a.KY, a.H - iy0));
        cols[i] = bit_range(max(0, -ix0), min(a.KX, a.W - ix0));
        if ((lane & 3) == 0) sOutOff[r] = (int64_t)n * a.out_sn + (int64_t)(a.y0 + by) * a.out_sh + (int64_t)(a.x0 + bx) * a.out_sw;
    }
    const uint8_t* const fillp = &g_fill.b[a.fill_raw][pj * 16];
    if (tid < BN) sWsum[tid] = 0;
    if (tid == 0) sFlags = 0;

    // scalar walk over (kernel row, kernel column, 64-byte channel chunk); additions only
    int32_t it_ky = 0, it_kx = 0, it_c64 = 0;
    int64_t it_off = 0, tap_off = 0, w_off = 0;
    // Request one step's operands into ring slot `slot` (uniform).
    auto request = [&](int slot) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            uint8_t* const st = sT + slot * STAGE + c * CHUNK + wave * 1024;
#pragma unroll
            for (int i = 0; i < NA; ++i)
                load_to_lds_16(wsrc[i] + w_off + 64 * c, st + NW * i * 1024);
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const uint8_t* src = bsrc[i] + it_off + 64 * c;
                if (!w.inside) src = ((rows[i] >> it_ky) & (cols[i] >> it_kx) & 1u) ? src : fillp;
                load_to_lds_16(src, st + (ABLK + NW * i) * 1024);
            }
        }
        w_off += 64 * KC;
        it_off += 64 * KC;
        it_c64 += KC;
        if (it_c64 == w.nc64) {
            it_c64 = 0;
            tap_off += a.in_sw;
            if (++it_kx == a.KX) {
                it_kx = 0;
                ++it_ky;
                tap_off += w.row_adv;
            }
            it_off = tap_off;
        }
    };

    const int S = w.nsteps;
    __syncthreads();  // (sOutOff, sWsum, sFlags are in place; no full barrier until the reduction is over)
    // NS - 1 steps in flight before the first is consumed.
#pragma unroll
    for (int j = 0; j < NS - 1; ++j) {
        if (j < S) request(j);
    }
    // the table rows of the workgroup's channels travel while the first operands do
    int32_t tw2 = 0, tbias = 0;
    if (tid < noc) {
        const int32_t* trow = a.table + (int64_t)(oc0 + tid) * a.table_stride;
        tw2 = trow[2];
        tbias = trow[3];
    }

    // operand reads: lane (c16, q) reads row c16 of a fragment, piece q
    const int frag_off = c16 * 64 + (((lane >> 4) ^ swz(c16)) << 4);
    const int a_rd = (wn * TN) * 1024 + frag_off;
    const int b_rd = BN * 64 + (wm * TM) * 1024 + frag_off;

    v4i acc[TN][TM];
    v4i wsa[TN];  // weight sums (input zero point away from the storage offset only)
#pragma unroll
    for (int f = 0; f < TN; ++f) {
        wsa[f] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int x = 0; x < TM; ++x) acc[f][x] = v4i{0, 0, 0, 0};
    }
    const int axor = (int)a.a_xor, wxor = (int)a.w_xor;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

    // The reduction loop, compiled twice: with and without the weight sums.
    auto reduce = [&](auto with_sums) {
        constexpr bool WS = decltype(with_sums)::value;
        int slot = 0;  // ring slot of step s
        for (int s = 0; s < S; ++s) {
            // The requests of step s are this wave's oldest; younger ones (at most NS - 2 steps) may stay in flight.
            // Near the end fewer are younger, so there everything is waited for.
            if (s + NS - 1 <= S) __builtin_amdgcn_s_waitcnt(vmcnt_imm((NS - 2) * (NA + NB) * KC));
            else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            // Every wave's pieces of step s are in LDS, and every wave has left step s - 1's slot. (The bare barrier:
            // __syncthreads() would first wait for ALL outstanding loads, which empties the ring at every step.)
            __builtin_amdgcn_s_barrier();
            if (s + NS - 1 < S) request(slot == 0 ? NS - 1 : slot - 1);
            const uint8_t* const st = sT + slot * STAGE;
            v4i fa[KC][TN], fb[KC][TM];
#pragma unroll
            for (int c = 0; c < KC; ++c) {
#pragma unroll
                for (int f = 0; f < TN; ++f) fa[c][f] = *reinterpret_cast<const v4i*>(st + c * CHUNK + a_rd + f * 1024);
#pragma unroll
                for (int x = 0; x < TM; ++x) fb[c][x] = *reinterpret_cast<const v4i*>(st + c * CHUNK + b_rd + x * 1024);
            }
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                if (wxor != 0) {  // uniform
#pragma unroll
                    for (int f = 0; f < TN; ++f) fa[c][f] ^= wxor;
                }
#pragma unroll
                for (int x = 0; x < TM; ++x) fb[c][x] ^= axor;
#pragma unroll
                for (int f = 0; f < TN; ++f)
#pragma unroll
                    for (int x = 0; x < TM; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[c][f], fb[c][x], acc[f][x], 0, 0, 0);
                if constexpr (WS) {
#pragma unroll
                    for (int f = 0; f < TN; ++f) wsa[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[c][f], ones, wsa[f], 0, 0, 0);
                }
            }
            slot = slot == NS - 1 ? 0 : slot + 1;
        }
    };
    if (a.da != 0) reduce(std::true_type{});
    else reduce(std::false_type{});
    __syncthreads();

    // ---- per-channel constants (thread = channel), as in the weights-resident kernel -----------------------
    if (a.da != 0 && wm == 0 && c16 == 0) {
        // every column of a sum fragment holds the same sums: lane (0, q) publishes rows 4q .. 4q + 3
#pragma unroll
        for (int f = 0; f < TN; ++f)
#pragma unroll
            for (int r = 0; r < 4; ++r) sWsum[wn * CW + channel_of_frag_row<TN>(f, 4 * (lane >> 4) + r)] = wsa[f][r];
    }
    const int64_t acc_bound = min((int64_t)a.ktot * 65025, (int64_t)2147483648LL);
    if (tid < BN) {
        const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
        const bool bad = shift > kMaxF64Shift;
        const bool sat = ppe_may_saturate(acc_bound, tbias, mult, shift);
        bool hi_bad = false;
        if (tid < noc) {
            hi_bad = shift < 1 || shift > 32 || ((int64_t)mult << (32 - min(shift, 32))) > 0x7fffffffLL;
            const double cb = ((__builtin_fabs((double)tbias) + 4294967296.0) * (double)mult + 2147483648.0 + 384.0 * __builtin_ldexp(1.0, shift));
            hi_bad = hi_bad || __builtin_ldexp(cb, 32 - shift) >= 4611686018427387904.0;
        }
        const int wf = (bad ? 1 : 0) | (sat ? 2 : 0) | (hi_bad ? 4 : 0);
        if (wf) atomicOr(&sFlags, wf);
        sW2[tid] = tw2;
        sBias[tid] = tbias;
    }
    __syncthreads();
    const int flags = sFlags;
    const PpeF64 pu = ppe_f64_setup(a.ppe, (flags & 2) != 0);
    int pmode = ppe_mode_of(pu, (flags & 1) != 0);
    if (pmode == PPE_MODE_FOLDED && !(flags & 4)) pmode = PPE_MODE_HI;
    EpiPack ep = epi_pack_setup(pu);
    if (pmode == PPE_MODE_SLOPE && !(flags & 4)) {
        // slope = pm * 2^-ps with |slope| <= 1 in this mode; the high-word form needs slope * 2^32 in int32
        const int32_t pm = a.ppe.prelu_mult, ps = a.ppe.prelu_shift;
        if (ps <= 32 && (ps >= 1 || pm == 0)) {
            const int64_t q = (int64_t)pm * ((int64_t)1 << (32 - ps));
            if (q >= -0x7fffffffLL && q <= 0x7fffffffLL) {
                const int64_t zpf = pu.zp + (ep.flip ? 128 : 0);
                const int64_t half = ps >= 1 ? (int64_t)1 << (ps - 1) : 0;
                pmode = PPE_MODE_HI_SLOPE;
                ep.pmq = __builtin_amdgcn_readfirstlane((int32_t)q);
                ep.cpz = (half + zpf * ((int64_t)1 << ps) - zpf * pm) * ((int64_t)1 << (32 - ps));
            }
        }
    }
    if (tid < BN) {
        const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
        const int32_t corr = a.da * sWsum[tid];  // |da| <= 255, |sum w'| < 2^23
        const double M = ppe_scale_M(mult, shift);
        double B = __builtin_fma((double)corr, M, ppe_scale_B(tbias, M, shift, a.ppe.round_mode));
        if (pmode != PPE_MODE_INT) B += ep.zp_fold;  // floor(x + zp) = floor(x) + zp
        sM[tid] = M;
        sBfull[tid] = B;
        sCorr[tid] = corr;
        if (pmode == PPE_MODE_HI || pmode == PPE_MODE_HI_SLOPE) {
            int32_t mq = 0;
            int64_t cq = 0;
            if (tid < noc) {
                const int64_t base = ((int64_t)tbias + corr) * mult + ((int64_t)1 << (shift - 1)) + ((int64_t)(pu.zp + (ep.flip ? 128 : 0)) << shift);
                mq = (int32_t)((uint32_t)mult << (32 - shift));
                cq = (int64_t)((uint64_t)base << (32 - shift));
            }
            sCorr[tid] = mq;
            reinterpret_cast<int64_t*>(sBfull)[tid] = cq;
        }
    }
    __syncthreads();

    // ---- PPE + store: this wave's CW channels of its 16 * TM pixels ---------------------------------------
    uint8_t* dst[TM];
    bool valid[TM];
    int32_t dws[TM];
#pragma unroll
    for (int x = 0; x < TM; ++x) {
        const int r = (wm * TM + x) * 16 + c16;
        valid[x] = m0 + r < a.M;
        dst[x] = a.out + sOutOff[r] + (int64_t)(oc0 + wn * CW) * a.out_sc;
        dws[x] = 0;
    }
    const int q = lane >> 4;
    const int nocw = noc - wn * CW;
    const EpiSmem ew = {sM + wn * CW, nullptr, sW2 + wn * CW, sBias + wn * CW, nullptr, nullptr};
    const double* const bw = sBfull + wn * CW;
    const int32_t* const cw = sCorr + wn * CW;
    uint4 other[FZ ? TM : 1];
    if constexpr (FZ) {
        if (nocw > 0) {  // uniform per wave; lanes past the last channel read a duplicate inside the tensor
            const int ch0 = min(16 * q, nocw - 16);
#pragma unroll
            for (int x = 0; x < TM; ++x) other[x] = *reinterpret_cast<const uint4*>(w.fz.other + ((dst[x] + ch0) - a.out));
        }
    }
    if (pmode == PPE_MODE_HI) wres_epilogue<TN, TM, PPE_MODE_HI, FZ>(a, ew, bw, cw, acc, dws, q, nocw, dst, valid, pu, ep, &w.fz, other);
    else if (pmode == PPE_MODE_HI_SLOPE) wres_epilogue<TN, TM, PPE_MODE_HI_SLOPE, FZ>(a, ew, bw, cw, acc, dws, q, nocw, dst, valid, pu, ep, &w.fz, other);
    else if (pmode == PPE_MODE_FOLDED) wres_epilogue<TN, TM, PPE_MODE_FOLDED, FZ>(a, ew, bw, cw, acc, dws, q, nocw, dst, valid, pu, ep, &w.fz, other);
    else if (pmode == PPE_MODE_SLOPE) wres_epilogue<TN, TM, PPE_MODE_SLOPE, FZ>(a, ew, bw, cw, acc, dws, q, nocw, dst, valid, pu, ep, &w.fz, other);
    else wres_epilogue<TN, TM, PPE_MODE_INT, FZ>(a, ew, bw, cw, acc, dws, q, nocw, dst, valid, pu, ep, &w.fz, other);
}

template <int WM, int WN, int TM, int TN, int NS, int KC = 1>
hipError_t launch_shape(TiledArgs& w, bool fused, hipStream_t stream) {
    constexpr int BM = 16 * TM * WM;
    constexpr int BN = 16 * TN * WN;
    constexpr size_t lds = (size_t)NS * (BM + BN) * 64 * KC;
    const ConvArgs& a = w.a;
    if (w.nc64 % KC != 0) return hipErrorNotSupported;
    w.nsteps = a.KY * a.KX * (w.nc64 / KC);
    w.ntm = (uint32_t)(((int64_t)a.M + BM - 1) / BM);
    w.ntn = (uint32_t)((a.bc + BN - 1) / BN);
    const uint64_t total = (uint64_t)w.ntm * w.ntn;
    if (total > 0x7ffffff0ull) return hipErrorNotSupported;
    const dim3 grid(xcd_grid((uint32_t)total)), block(64 * WM * WN);
    if (fused) {
        if constexpr (TN == 4) {
            auto kernel = &conv_tiled_kernel<WM, WN, TM, TN, NS, KC, true>;
            static LdsGrant grant;
            if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
            return emit(kernel, grid, block, lds, stream, w);
        }
        return hipErrorNotSupported;
    }
    auto kernel = &conv_tiled_kernel<WM, WN, TM, TN, NS, KC, false>;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    return emit(kernel, grid, block, lds, stream, w);
}

}  // namespace

// Shapes: 1 = 128 px x 128 ch (4 waves), 2 = 64 px x 128 ch (4 waves), 3 = 256 px x 128 ch (8 waves),
// 4 = 128 px x 64 ch (4 waves), 5 = shape 1 with steps of 128 bytes of the reduction (input channels a multiple of 128),
// 6 = shape 5 as eight waves of 32 px x 64 ch, two workgroups = sixteen waves per CU. shape 0 = automatic.
hipError_t launch_conv_tiled(const ConvArgs& a, hipStream_t stream, int shape, const FuseAdd* fuse) {
    if (a.IC % 64 != 0 || a.dw != 0 || a.KY > 32 || a.KX > 32) return hipErrorNotSupported;
    if (a.M > 0x7fffffff - 1024) return hipErrorNotSupported;
    if (fuse != nullptr && a.out_sc != 1) return hipErrorNotSupported;
    TiledArgs w;
    memset(&w, 0, sizeof(w));
    w.a = a;
    w.a.fill_raw = (a.fill ^ a.a_xor) & 0xFFu;
    if (fuse) w.fz = *fuse;
    w.nc64 = a.IC / 64;
    w.nsteps = a.KY * a.KX * w.nc64;
    w.row_adv = a.in_sh - (int64_t)a.KX * a.in_sw;
    const int64_t iy_lo = (int64_t)a.y0 * a.SY - a.PT, iy_hi = (int64_t)(a.y0 + a.bh - 1) * a.SY - a.PT + a.KY - 1;
    const int64_t ix_lo = (int64_t)a.x0 * a.SX - a.PL, ix_hi = (int64_t)(a.x0 + a.bw - 1) * a.SX - a.PL + a.KX - 1;
    w.inside = iy_lo >= 0 && iy_hi < a.H && ix_lo >= 0 && ix_hi < a.W;
    if (shape == 0) {
        // The largest tile that still gives every CU about two workgroups.
        const auto groups = [&](int bm, int bn) { return (((int64_t)a.M + bm - 1) / bm) * ((a.bc + bn - 1) / bn); };
        shape = groups(128, 128) >= 512 ? (a.IC % 128 == 0 ? 6 : 1) : 2;
    }
    const bool fz = fuse != nullptr;
    switch (shape) {
    case 1: return launch_shape<2, 2, 4, 4, 4>(w, fz, stream);
    case 2: return launch_shape<2, 2, 2, 4, 4>(w, fz, stream);
    case 3: return launch_shape<4, 2, 4, 4, 3>(w, fz, stream);
    case 4: return launch_shape<2, 2, 4, 2, 4>(w, fz, stream);
    case 5: return launch_shape<2, 2, 4, 4, 2, 2>(w, fz, stream);
    case 6: return launch_shape<4, 2, 2, 4, 2, 2>(w, fz, stream);
    default: return hipErrorNotSupported;
    }
}

}  // namespace nce
