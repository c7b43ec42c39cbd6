// CONV task, patch kernel: implicit GEMM on v_mfma_i32_16x16x64_i8 with BOTH operands read from LDS and every input byte
// fetched from memory once per workgroup - for kernels larger than 1x1, where the other kernels fetch an input pixel
// once per tap (nine times for 3x3) and are bound by the CU's load path (the weights-resident kernel) or by the
// L2-to-LDS stream (the LDS-tiled kernel).
//
// A workgroup of eight waves owns a slice of 16 * NF output channels and walks patches of the output: PR consecutive
// output rows of one image, all columns of the box. Per workgroup, once: the slice's weights for the whole reduction go
// to LDS as 1 KiB blocks of 16 rows x 64 bytes (block = reduction step x channel fragment). Per patch: the input pixels
// the patch's windows touch - (PR - 1) * SY + KY rows of (bw - 1) * SX + KX pixels, all IC channels: the patch plus its
// halo - go to LDS, pixels outside the image as a line of the input zero point, so that no tap needs a mask. Both
// transfers are global_load_lds_dwordx4 (no registers); a wave then re-biases the blocks it fetched itself in place
// (u8 -> i8, x ^ 0x80: once per byte instead of once per use) and the workgroup passes one barrier. From there a wave
// works alone on groups of NPX pixel fragments (16 consecutive pixels of the patch in row-major order each): per
// reduction step (tap, 64 input channels) it reads NF weight fragments and NPX activation fragments with ds_read_b128 and
// issues NF * NPX matrix instructions - 0.5 KiB of LDS reads per instruction for NF = NPX = 4, half of what the
// LDS pipe sustains at the full matrix rate. With room for two patches in LDS the next patch's pixels are requested
// before the current one is computed.
//
// Where a pixel's pieces sit: a ds_read_b128 is served in four clocks, sixteen lanes each (nce_conv_lds.h), and the
// operand read gives a set of sixteen lanes all sixteen pixels of a fragment - pixels 0-3 and 12-15 with 16-byte piece q
// of the step, pixels 4-11 with piece q ^ 1. Pixels are stored at slot * IC (slot = halo row * pitch + halo column); a
// pixel's IC / 16 pieces are permuted by a key that is consecutive for consecutive pixels of a fragment (key = halo
// row * bw + halo column; the pitch is padded to bw modulo 8 where a pixel is narrower than the 256 bytes the banks
// span, so that slot and key agree modulo 8 across the row ends a fragment crosses): within each window of U = min(IC /
// 16, 16) pieces, odd pieces take the upper half of the positions and even pieces the lower half, and inside a half piece
// 2 j + b sits at ((key >> (4 - log2 U)) + j) mod (U / 2). Then the eight pixels a set reads with an even piece differ in
// that sum, likewise the eight it reads with an odd piece, and every read runs at 256 bytes per clock (checked against
// the measured lane sets for every fragment, tap and chunk of the shapes this kernel takes).
//
// Conditions (host): stride 1, input channels 64, 128, 256, 512 or 1024, weights zero point equal to their storage offset,
// weights slice + one patch within the LDS. Semantics and the fused PPE are those of the other convolution kernels
// (nce_conv_epi.h).
#include "nce_conv_epi.h"
#include "nce_conv_lds.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace nce {

namespace {

using namespace wres_detail;
using namespace lds_detail;

constexpr size_t kPatchLdsCap = 156 * 1024;  // dynamic LDS a workgroup may ask for (the per-channel tables are static)

struct PatchArgs {
    ConvArgs a;
    int32_t PR;         // output rows per patch
    int32_t nrp;        // patches per image: ceil(bh / PR)
    uint32_t npatch;    // images x nrp
    uint32_t ngroups;   // workgroups per channel slice
    uint32_t tpg;       // patches per workgroup
    uint32_t nslices;   // channel slices of 16 * NF
    int32_t pitch;      // slots per halo row
    int32_t hcols;      // halo columns: (bw - 1) * SX + KX
    int32_t nblk;       // 1 KiB blocks of one patch's pixels in LDS
    int32_t nsteps;     // 64-byte reduction steps: KY * KX * IC / 64
    int32_t nc64;       // 64-byte chunks along IC
    int32_t ulog_full;  // log2(IC / 16)
    int32_t nbuf;       // 1 or 2 patch buffers
    uint32_t halo_bytes;  // bytes of one patch buffer (nblk KiB)
    FastDiv div_nrp, div_pitch;
#ifdef PATCH_TRACE
    uint64_t* trace;  // probe builds only: [workgroup][wave][32] timestamps (100 MHz)
#endif
};

#ifdef PATCH_TRACE
static uint64_t* g_probe_trace = nullptr;  // set by the probe program before it launches
#define PATCH_MARK(i)                                                                                                  \
    do {                                                                                                               \
        if (lane == 0 && (i) < 32) w.trace[((size_t)blockIdx.x * 16 + wave) * 32 + (i)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#define PATCH_MARK_DECL int patch_mark = 4
#define PATCH_MARK_SEQ()  \
    do {                  \
        PATCH_MARK(patch_mark); \
        ++patch_mark;     \
    } while (0)
#else
#define PATCH_MARK(i) do { } while (0)
#define PATCH_MARK_DECL do { } while (0)
#define PATCH_MARK_SEQ() do { } while (0)
#endif

// Position (in 16-byte units from the pixel's first byte) of piece `piece` of the pixel with key `key`. ULOG = log2 of
// the window: min(IC / 16, 16) pieces.
template <int ULOG>
__device__ __forceinline__ int halo_pos(int key, int piece) {
    constexpr int H = 1 << (ULOG - 1);
    constexpr int S = 4 - ULOG;
    const int pl = piece & ((1 << ULOG) - 1);
    return (piece & ~15) | (H * (pl & 1) + (((key >> S) + (pl >> 1)) & (H - 1)));
}
// ... and the piece that sits at position `pos`.
template <int ULOG>
__device__ __forceinline__ int halo_piece(int key, int pos) {
    constexpr int H = 1 << (ULOG - 1);
    constexpr int S = 4 - ULOG;
    const int pp = pos & ((1 << ULOG) - 1);
    const int j = ((pp & (H - 1)) - (key >> S)) & (H - 1);
    return (pos & ~15) | (2 * j + (pp >> (ULOG - 1)));
}

// NW waves per workgroup: 8 with groups of NPX = 4 pixel fragments (two waves per SIMD, 256 registers each), or 16 with
// groups of NPX = 2 (four waves per SIMD, 128 registers each: more waves to fill the matrix unit while others run their
// epilogues or stand at a request, at 0.75 instead of 0.5 KiB of LDS reads per matrix instruction).
template <int NF, int NPX, int ULOG, int NW>
__global__ __launch_bounds__(64 * NW, NW / 4) void conv_patch_kernel(PatchArgs w) {
    prefetch_kernel_arguments<sizeof(PatchArgs)>();
    constexpr int BN = 16 * NF;
    const ConvArgs& a = w.a;

    extern __shared__ __attribute__((aligned(16))) uint8_t sL[];  // weights [nsteps][NF] KiB, then nbuf patch buffers
    __shared__ int32_t sW2[BN], sBias[BN], sWsum[BN];
    __shared__ int32_t sCorr[BN];     // integer path: da * sum of weights; high-word path: scaled multiplier
    __shared__ double sM[BN], sBfull[BN];
    __shared__ int32_t sFlags;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;

    const uint32_t ntotal = w.ngroups * w.nslices;
    const uint32_t lid = xcd_tile(blockIdx.x, ntotal);
    if (lid >= ntotal) return;  // uniform for the whole workgroup
    // slices innermost: the workgroups of one XCD share patches (whose pixels then come out of one L2 for all slices)
    const uint32_t group = lid / w.nslices, slice = lid - group * w.nslices;
    const int32_t oc0 = a.z0 + (int32_t)slice * BN;
    const int32_t noc = min(BN, a.z0 + a.bc - oc0);
    const uint32_t p_begin = group * w.tpg;
    const uint32_t p_end = min(p_begin + w.tpg, w.npatch);
    if (p_begin >= p_end) return;  // uniform

    PATCH_MARK(0);
#ifdef PATCH_PRIO
    // The lower half of the waves (one or two per SIMD) outranks the upper half at instruction issue: where both are in
    // their reductions the lower one gets the matrix unit and finishes at full speed, and the upper one runs its
    // reduction while the lower one is in its epilogue - the two fall into opposite phases by themselves.
    if (wave < NW / 2) __builtin_amdgcn_s_setprio(3);
#endif
    const int wbytes = w.nsteps * NF * 1024;
    uint8_t* const sHalo = sL + wbytes;
    const int IC = a.IC;
    const int axor = (int)a.a_xor, wxor = (int)a.w_xor;

    if (tid < BN) sWsum[tid] = 0;
    __syncthreads();

    // ---- requests -------------------------------------------------------------------------------------------------------
    // The last wave fetches nothing: it reads the table rows of the slice's channels (lane = channel) and derives the
    // per-channel constants while the other waves' requests travel (a request is accepted only as fast as the memory
    // delivers, so one wave less does not slow the transfer down).
    constexpr int NL = NW - 1;
    const bool consts_wave = wave == NL;
    // Weights: block wb = step * NF + fragment; lane 4 r + j fetches the piece that belongs at position j of row r.
    const int prow = lane >> 2;
    const int pj = (lane & 3) ^ swz(prow);
    const int nwblk = w.nsteps * NF;
    // Pixels of patch pt into buffer `buf`: block k holds the slots k * (1024 / IC) ...; a lane fetches the piece that
    // belongs at its position of its slot's pixel, or the same piece of the zero-point line for a slot outside the image
    // (or beyond the patch's own rows and columns).
    const uint8_t* const fillp = &g_fill.b[a.fill_raw][0];
    const int lane_slot = lane >> w.ulog_full, lane_pos = lane & ((1 << w.ulog_full) - 1);
    // Parameters of one patch's requests (uniform), and the request of one block.
    struct PatchSrc {
        const uint8_t* img;  // address of halo slot (0, 0)'s pixel (may lie outside the image)
        int32_t iy_lo, iy_n, ix_lo, ix_n;  // halo rows and columns that exist for this patch and lie inside the image
        uint8_t* dst;        // the patch buffer
    };
    auto patch_src = [&](uint32_t pt, int buf) {
        PatchSrc ps;
        const int32_t n = (int32_t)fdiv(pt, w.div_nrp);
        const int32_t row0 = ((int32_t)pt - n * w.nrp) * w.PR;
        const int32_t rows = min(w.PR, a.bh - row0);
        const int32_t gy0 = (a.y0 + row0) * a.SY - a.PT, gx0 = a.x0 * a.SX - a.PL;
        ps.iy_lo = max(0, -gy0);
        ps.iy_n = min((rows - 1) * a.SY + a.KY, a.H - gy0) - ps.iy_lo;
        ps.ix_lo = max(0, -gx0);
        ps.ix_n = min(w.hcols, a.W - gx0) - ps.ix_lo;
        ps.img = a.in + (int64_t)n * a.in_sn + (int64_t)gy0 * a.in_sh + (int64_t)gx0 * a.in_sw;
        ps.dst = sHalo + (uint32_t)buf * w.halo_bytes;
        return ps;
    };
    const int32_t in_sh32 = (int32_t)a.in_sh, in_sw32 = (int32_t)a.in_sw;  // (an image's extent fits 31 bits: host)
    auto request_block = [&](const PatchSrc& ps, int k) {
        const int slot = (k << (6 - w.ulog_full)) + lane_slot;
        const int iy = (int)fdiv((uint32_t)slot, w.div_pitch);
        const int ix = slot - iy * w.pitch;
        const int piece = halo_piece<ULOG>(iy * a.bw + ix, lane_pos);
        const bool inside = (uint32_t)(iy - ps.iy_lo) < (uint32_t)ps.iy_n && (uint32_t)(ix - ps.ix_lo) < (uint32_t)ps.ix_n;
        const uint8_t* src = inside ? ps.img + (iy * in_sh32 + ix * in_sw32 + piece * 16) : fillp + (piece & 3) * 16;
        load_to_lds_16(src, ps.dst + k * 1024);
    };
    // (first, stride): which blocks of a patch this wave fetches - and later re-biases, after its own requests have landed
    auto request_patch = [&](uint32_t pt, int buf, int first, int stride) {
        const PatchSrc ps = patch_src(pt, buf);
        for (int k = first; k < w.nblk; k += stride) request_block(ps, k);
    };
    auto rebias_patch = [&](int buf, int first, int stride) {
        if (axor == 0) return;  // uniform
        uint8_t* const dstb = sHalo + (uint32_t)buf * w.halo_bytes + lane * 16;
        // four blocks at a time: read, XOR and write back one by one, a wave pays one LDS round trip per block
        int k = first;
        for (; k + 3 * stride < w.nblk; k += 4 * stride) {
            v4i* const p0 = reinterpret_cast<v4i*>(dstb + k * 1024);
            v4i* const p1 = reinterpret_cast<v4i*>(dstb + (k + stride) * 1024);
            v4i* const p2 = reinterpret_cast<v4i*>(dstb + (k + 2 * stride) * 1024);
            v4i* const p3 = reinterpret_cast<v4i*>(dstb + (k + 3 * stride) * 1024);
            const v4i v0 = *p0, v1 = *p1, v2 = *p2, v3 = *p3;
            *p0 = v0 ^ axor;
            *p1 = v1 ^ axor;
            *p2 = v2 ^ axor;
            *p3 = v3 ^ axor;
        }
        for (; k < w.nblk; k += stride) {
            v4i* const p = reinterpret_cast<v4i*>(dstb + k * 1024);
            *p = *p ^ axor;
        }
    };
    const int64_t acc_bound = min((int64_t)a.ktot * 65025, (int64_t)2147483648LL);
    if (consts_wave) {
        int32_t tw2 = 0, tbias = 0;
        if (lane < noc) {
            const int32_t* trow = a.table + (int64_t)(oc0 + lane) * a.table_stride;
            tw2 = trow[2];
            tbias = trow[3];
        }
        const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
        const bool bad = lane < BN && shift > kMaxF64Shift;
        const bool sat = lane < BN && ppe_may_saturate(acc_bound, tbias, mult, shift);
        bool hi_bad = false;
        if (lane < noc) {
            hi_bad = shift < 1 || shift > 32 || ((int64_t)mult << (32 - min(shift, 32))) > 0x7fffffffLL;
            const double cb = ((__builtin_fabs((double)tbias) + 4294967296.0) * (double)mult + 2147483648.0 + 384.0 * __builtin_ldexp(1.0, shift));
            hi_bad = hi_bad || __builtin_ldexp(cb, 32 - shift) >= 4611686018427387904.0;
        }
        const int wf = (__any(bad) ? 1 : 0) | (__any(sat) ? 2 : 0) | (__any(hi_bad) ? 4 : 0);
        if (lane == 0) sFlags = wf;
        if (lane < BN) {
            const double M = ppe_scale_M(mult, shift);
            sW2[lane] = tw2;
            sBias[lane] = tbias;
            sM[lane] = M;
            sBfull[lane] = ppe_scale_B(tbias, M, shift, a.ppe.round_mode);
        }
    } else {
        for (int wb = wave; wb < nwblk; wb += NL) {
            const int s = wb / NF, f = wb - s * NF;
            const int ch = min(channel_of_frag_row<NF>(f, prow), noc - 1);  // rows past the box's last channel duplicate it (not stored)
            const uint8_t* src = a.w + (int64_t)(oc0 + ch) * a.w_soc + s * 64 + pj * 16;
            load_to_lds_16(src, sL + wb * 1024);
        }
        request_patch(p_begin, 0, wave, NL);
        PATCH_MARK(1);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        PATCH_MARK(2);
        // weights: re-bias u8 storage; the per-channel sums of the re-biased weights when the input zero point is not the
        // storage offset (each lane adds up the piece it fetched; the four lanes of a row combine)
        if (wxor != 0 || a.da != 0) {
            for (int wb = wave; wb < nwblk; wb += NL) {
                v4i* const p = reinterpret_cast<v4i*>(sL + wb * 1024 + lane * 16);
                v4i v = *p;
                if (wxor != 0) {
                    v = v ^ wxor;
                    *p = v;
                }
                if (a.da != 0) {
                    const int f = wb % NF;
                    int32_t sum = bytesum(make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]));
                    sum += __shfl_xor(sum, 1);
                    sum += __shfl_xor(sum, 2);
                    if ((lane & 3) == 0) atomicAdd(&sWsum[channel_of_frag_row<NF>(f, prow)], sum);
                }
            }
        }
        rebias_patch(0, wave, NL);
    }
    __syncthreads();  // weights, first patch, weight sums and the constants' first part complete

    // ---- per-channel constants (thread = channel), as in the other MFMA kernels ----------------------------------------
    const int flags = sFlags;
    const PpeF64 pu = ppe_f64_setup(a.ppe, (flags & 2) != 0);
    int pmode = ppe_mode_of(pu, (flags & 1) != 0);
    if (pmode == PPE_MODE_FOLDED && !(flags & 4)) pmode = PPE_MODE_HI;
    EpiPack ep = epi_pack_setup(pu);
    if (pmode == PPE_MODE_SLOPE && !(flags & 4)) {
        // slope = pm * 2^-ps with |slope| <= 1 in this mode; the high-word form needs slope * 2^32 in int32
        const int32_t pm = a.ppe.prelu_mult, ps = a.ppe.prelu_shift;
        if (ps <= 32 && (ps >= 1 || pm == 0)) {
            const int64_t qq = (int64_t)pm * ((int64_t)1 << (32 - ps));
            if (qq >= -0x7fffffffLL && qq <= 0x7fffffffLL) {
                const int64_t zpf = pu.zp + (ep.flip ? 128 : 0);
                const int64_t half = ps >= 1 ? (int64_t)1 << (ps - 1) : 0;
                pmode = PPE_MODE_HI_SLOPE;
                ep.pmq = __builtin_amdgcn_readfirstlane((int32_t)qq);
                ep.cpz = (half + zpf * ((int64_t)1 << ps) - zpf * pm) * ((int64_t)1 << (32 - ps));
            }
        }
    }
    // (This kernel keeps two epilogues: the high-word integer forms for the usual shifts, and the 64-bit integer
    // reference form for everything else - the FP64 forms of the other kernels would be two more copies of the epilogue.)
    if (pmode != PPE_MODE_HI && pmode != PPE_MODE_HI_SLOPE) pmode = PPE_MODE_INT;
    if (tid < BN) {
        const int32_t tw2 = sW2[tid], tbias = sBias[tid];
        const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
        const int32_t corr = a.da * sWsum[tid];  // |da| <= 255, |sum w'| < 2^23
        double B = __builtin_fma((double)corr, sM[tid], sBfull[tid]);
        if (pmode != PPE_MODE_INT) B += ep.zp_fold;  // floor(x + zp) = floor(x) + zp
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
    const EpiSmem ew = {sM, nullptr, sW2, sBias, nullptr, nullptr};
    PATCH_MARK(3);
    PATCH_MARK_DECL;

    // ---- operand reads ------------------------------------------------------------------------------------------------------
    // weights: lane (c16, q) reads piece q of row c16 of a block
    const int wfrag_off = c16 * 64 + ((q ^ swz(c16)) << 4);
    constexpr int H = 1 << (ULOG - 1);
    constexpr int S = 4 - ULOG;
    constexpr int POSMASK = (H - 1) << 4;
    // Position of this lane's piece inside its half of a window, as a byte offset: bits S .. S + ULOG - 2 of
    // (key + (piece >> 1 << S)), moved up to bit 4: one addition of a per-step scalar to a per-lane constant and one AND.
    const int hq = (H * (q & 1)) << 4;  // byte offset of this lane's half of a window
    const int32_t out_sh32 = (int32_t)a.out_sh, out_sw32 = (int32_t)a.out_sw;  // (a patch's extent fits 31 bits: host)

    for (uint32_t pt = p_begin; pt < p_end; ++pt) {
        const int buf = w.nbuf == 2 ? (int)((pt - p_begin) & 1u) : 0;
        const bool more = pt + 1 < p_end;
        // With two buffers every wave requests its share of the NEXT patch's blocks one at a time between the steps of
        // its first reduction of this patch: a request is accepted only as fast as the memory delivers and a wave may
        // have few in flight (from HBM, eight waves requesting at once stand still for about as long as the transfer
        // takes and four for twice as long), so the requests are spread out and the matrix instructions run on.
        // (The other buffer was last read for patch pt - 1, which every wave left before the barrier that ended it.)
        const bool ahead = w.nbuf == 2 && more;
        PatchSrc nx = {};
        if (ahead) nx = patch_src(pt + 1, buf ^ 1);
        const int req_first = wave, req_stride = NW;  // this wave's blocks of the next patch
        int kreq = ahead ? req_first : w.nblk;  // this wave's next block to request
        const uint8_t* const hb = sHalo + (uint32_t)buf * w.halo_bytes;
        const int32_t n = (int32_t)fdiv(pt, w.div_nrp);
        const int32_t row0 = ((int32_t)pt - n * w.nrp) * w.PR;
        const int32_t rows = min(w.PR, a.bh - row0);
        const int32_t npx = rows * a.bw;
        const int32_t ngr = (npx + 16 * NPX - 1) / (16 * NPX);
        uint8_t* const obase = a.out + (int64_t)n * a.out_sn + (int64_t)(a.y0 + row0) * a.out_sh + (int64_t)a.x0 * a.out_sw + (int64_t)oc0 * a.out_sc;
        // With two buffers the next patch's pixels are re-biased by the wave that fetched them as soon as that wave is
        // through its last reduction of this patch - ahead of its last epilogue, so that the wait covers the requests
        // (long landed) and not the stores that epilogue is about to issue.
        bool next_done = !ahead;
        auto finish_next = [&]() {
            for (; kreq < w.nblk; kreq += req_stride) request_block(nx, kreq);  // (what the reduction steps did not get to)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            rebias_patch(buf ^ 1, req_first, req_stride);
            next_done = true;
        };
        PATCH_MARK_SEQ();   // patch top (after the next patch's requests)
        for (int g = wave; g < ngr; g += NW) {
            PATCH_MARK_SEQ();   // group start
            // this lane's pixel of every fragment: LDS address of its slot (tap (0, 0), this lane's half) and its key
            int32_t abase[NPX], akq[NPX];
#pragma unroll
            for (int x = 0; x < NPX; ++x) {
                int32_t p = (g * NPX + x) * 16 + c16;
                // (a row past the patch's last pixel reads the pixel 16 k before it: the fragment keeps its bank pattern)
                if (p >= npx) p = max(p - 16 * (((p - npx) >> 4) + 1), 0);
                const int32_t y = (int32_t)fdiv((uint32_t)p, a.div_bw);
                const int32_t xx = p - y * a.bw;
                abase[x] = (y * a.SY * w.pitch + xx * a.SX) * IC + hq;
                akq[x] = (y * a.SY * a.bw + xx * a.SX + ((q >> 1) << S)) << (4 - S);
            }
            v4i acc[NF][NPX];

            // scalar walk over (kernel row, kernel column, 64-byte chunk); two register sets so that the reads of step
            // s + 1 are in flight while the matrix instructions of step s run
            int32_t it_ky = 0, it_kx = 0, it_c = 0;
            const uint8_t* wp = sL + wfrag_off;
            auto fetch = [&](v4i (&fa)[NF], v4i (&fb)[NPX]) {
                const int32_t tapoff = (it_ky * w.pitch + it_kx) * IC + ((it_c >> 2) << 8);
                const int32_t ts = (it_ky * a.bw + it_kx + ((2 * (it_c & 3)) << S)) << (4 - S);
#pragma unroll
                for (int f = 0; f < NF; ++f) fa[f] = *reinterpret_cast<const v4i*>(wp + f * 1024);
#pragma unroll
                for (int x = 0; x < NPX; ++x) fb[x] = *reinterpret_cast<const v4i*>(hb + (abase[x] + tapoff + ((akq[x] + ts) & POSMASK)));
                wp += NF * 1024;
                // (selects, no branches: between the reads of one step and the matrix instructions of the other the code
                // must stay one block, or the wait before those instructions also covers the reads just issued)
                ++it_c;
                const bool wrap_c = it_c == w.nc64;
                it_c = wrap_c ? 0 : it_c;
                it_kx += wrap_c ? 1 : 0;
                const bool wrap_x = it_kx == a.KX;
                it_kx = wrap_x ? 0 : it_kx;
                it_ky += wrap_x ? 1 : 0;
            };
            auto mma = [&](const v4i (&fa)[NF], const v4i (&fb)[NPX]) {
#pragma unroll
                for (int f = 0; f < NF; ++f)
#pragma unroll
                    for (int x = 0; x < NPX; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[f], fb[x], acc[f][x], 0, 0, 0);
            };
            const int Sn = w.nsteps;
            const v4i zero = {0, 0, 0, 0};
            auto request_one = [&]() {
#ifdef PATCH_KO_NOREQ
                if (false) {
#else
                if (kreq < w.nblk) {  // uniform
#endif
                    request_block(nx, kreq);
                    kreq += req_stride;
                }
            };
            if constexpr (NW == 8 || NF == 2) {
                // Two waves per SIMD (or registers to spare): two register sets, so that the reads of step s + 1 are in flight while the matrix
                // instructions of step s run. (Both requests of the loop body are unconditional and the tail is written out,
                // so that every block of matrix instructions follows the requests of the step after it on every path: the
                // wait before it then names just the older set, and the younger one stays in flight.)
                v4i fa0[NF], fb0[NPX], fa1[NF], fb1[NPX];
                // (Nothing but LDS reads may be outstanding on the LDS counter inside the loop: with a scalar load still
                // counted there - they return out of order - every wait in the loop would be a wait for everything.)
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                constexpr int kWaitOlderSet = 0xC07F | ((NF + NPX) << 8);  // lgkmcnt(NF + NPX): all but the reads of the newest step
                fetch(fa0, fb0);
                __builtin_amdgcn_sched_barrier(0);
                fetch(fa1, fb1);  // (unconditional, like every fetch here: a reduction of one step reads, and ignores, what follows)
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_waitcnt(kWaitOlderSet);
#pragma unroll
                for (int f = 0; f < NF; ++f)  // the first step starts the accumulators (no zeroing pass)
#pragma unroll
                    for (int x = 0; x < NPX; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa0[f], fb0[x], zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                int s = 1;
                for (; s + 2 < Sn; s += 2) {
                    // (the fences keep the compiler from sinking a step's reads to just above their use)
                    fetch(fa0, fb0);
                    request_one();
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_waitcnt(kWaitOlderSet);
                    mma(fa1, fb1);
                    __builtin_amdgcn_sched_barrier(0);
                    fetch(fa1, fb1);
                    request_one();
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_waitcnt(kWaitOlderSet);
                    mma(fa0, fb0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (s + 1 < Sn) {
                    fetch(fa0, fb0);
                    mma(fa1, fb1);
                    mma(fa0, fb0);
                } else if (s < Sn) {
                    mma(fa1, fb1);
                }
            } else {
                // Four waves per SIMD: one register set; the other waves cover this one's read latency.
                v4i fa0[NF], fb0[NPX];
                fetch(fa0, fb0);
#pragma unroll
                for (int f = 0; f < NF; ++f)
#pragma unroll
                    for (int x = 0; x < NPX; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa0[f], fb0[x], zero, 0, 0, 0);
                for (int s = 1; s < Sn; ++s) {
                    fetch(fa0, fb0);
                    request_one();
                    mma(fa0, fb0);
                }
            }
            PATCH_MARK_SEQ();   // reduction done (issued)
            if (!next_done && g + NW >= ngr) finish_next();
            PATCH_MARK_SEQ();   // next patch re-biased

            // ---- PPE + store -------------------------------------------------------------------------------------------------
            uint8_t* dst[NPX];
            bool valid[NPX];
            int32_t dws[NPX];
#pragma unroll
            for (int x = 0; x < NPX; ++x) {
                const int32_t p = (g * NPX + x) * 16 + c16;
                valid[x] = p < npx;
                const int32_t pc = min(p, npx - 1);
                const int32_t y = (int32_t)fdiv((uint32_t)pc, a.div_bw);
                const int32_t xx = pc - y * a.bw;
                dst[x] = obase + (y * out_sh32 + xx * out_sw32);
                dws[x] = 0;
            }
            if (pmode == PPE_MODE_HI) wres_epilogue<NF, NPX, PPE_MODE_HI>(a, ew, sBfull, sCorr, acc, dws, q, noc, dst, valid, pu, ep);
            else if (pmode == PPE_MODE_HI_SLOPE) wres_epilogue<NF, NPX, PPE_MODE_HI_SLOPE>(a, ew, sBfull, sCorr, acc, dws, q, noc, dst, valid, pu, ep);
            else wres_epilogue<NF, NPX, PPE_MODE_INT>(a, ew, sBfull, sCorr, acc, dws, q, noc, dst, valid, pu, ep);
            PATCH_MARK_SEQ();   // epilogue issued
        }
        if (more) {
            if (w.nbuf == 1) {
                __syncthreads();  // every wave has left the only buffer
                request_patch(pt + 1, 0, wave, NW);
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
                rebias_patch(0, wave, NW);
                __syncthreads();
            } else {
                if (!next_done) finish_next();  // (a wave without a group in this patch)
                // The next patch is complete and every wave has left this one. (The bare barrier: __syncthreads() would
                // also wait for the stores of the epilogue.)
                asm volatile("" ::: "memory");       // (no LDS access moves across the barrier at compile time)
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's re-biasing writes
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
        }
        PATCH_MARK_SEQ();       // patch end (after the barrier)
    }
}

template <int NF, int NPX, int ULOG, int NW>
hipError_t launch_patch(const PatchArgs& w, size_t lds, hipStream_t stream) {
    auto kernel = &conv_patch_kernel<NF, NPX, ULOG, NW>;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    const uint32_t total = w.ngroups * w.nslices;
    return emit(kernel, dim3(xcd_grid(total)), dim3(64 * NW), lds, stream, w);
}

template <int NF>
hipError_t launch_patch_u(const PatchArgs& w, size_t lds, int ulog, int waves, int npxf, hipStream_t stream) {
    if (waves == 16 && npxf == 1) {
        switch (ulog) {
        case 2: return launch_patch<NF, 1, 2, 16>(w, lds, stream);
        case 3: return launch_patch<NF, 1, 3, 16>(w, lds, stream);
        case 4: return launch_patch<NF, 1, 4, 16>(w, lds, stream);
        default: return hipErrorNotSupported;
        }
    }
    if (waves == 16) {
        switch (ulog) {
        case 2: return launch_patch<NF, 2, 2, 16>(w, lds, stream);
        case 3: return launch_patch<NF, 2, 3, 16>(w, lds, stream);
        case 4: return launch_patch<NF, 2, 4, 16>(w, lds, stream);
        default: return hipErrorNotSupported;
        }
    }
    switch (ulog) {
    case 2: return launch_patch<NF, 4, 2, 8>(w, lds, stream);
    case 3: return launch_patch<NF, 4, 3, 8>(w, lds, stream);
    case 4: return launch_patch<NF, 4, 4, 8>(w, lds, stream);
    default: return hipErrorNotSupported;
    }
}

}  // namespace

// nf_forced: 0 = automatic, 2 or 4 = channel fragments per slice; pr_forced: 0 = automatic, else output rows per patch;
// waves_forced: 0 = automatic, 8 or 16 = waves per workgroup (groups of four or two pixel fragments); npx_forced = 1 with 16
// waves: groups of one pixel fragment (small patches: a group per wave).
hipError_t launch_conv_patch(const ConvArgs& a, hipStream_t stream, int nf_forced, int pr_forced, int waves_forced, int npx_forced) {
    const int waves = waves_forced == 16 ? 16 : 8;
    const int npxf = waves == 16 ? (npx_forced == 1 ? 1 : 2) : 4;  // pixel fragments per group
    if (a.SY != 1 || a.SX != 1 || a.dw != 0) return hipErrorNotSupported;
    if (a.IC != 64 && a.IC != 128 && a.IC != 256 && a.IC != 512 && a.IC != 1024) return hipErrorNotSupported;
    if (a.KY > 16 || a.KX > 16 || a.bw > 4096 || a.bh > 32768) return hipErrorNotSupported;
    // (the kernel adds a pixel's offset inside its patch to the patch's address in 32 bits)
    if (a.in_sh < 0 || a.in_sw < 0 || (int64_t)(a.H + 32) * a.in_sh + (int64_t)(a.W + 32) * a.in_sw > 0x7fffffffLL) return hipErrorNotSupported;
    if (a.out_sh < 0 || a.out_sw < 0 || (int64_t)a.bh * a.out_sh + (int64_t)a.bw * a.out_sw > 0x7fffffffLL) return hipErrorNotSupported;
    PatchArgs w;
    memset(&w, 0, sizeof(w));
    w.a = a;
    w.a.fill_raw = (a.fill ^ a.a_xor) & 0xFFu;
    w.nc64 = a.IC / 64;
    w.nsteps = a.KY * a.KX * w.nc64;
    int ulf = 0;
    while ((16 << ulf) < a.IC) ++ulf;
    w.ulog_full = ulf;
    const int ulog = std::min(ulf, 4);
    w.hcols = (a.bw - 1) * a.SX + a.KX;
    w.pitch = w.hcols;
    if (a.IC < 256)
        while ((w.pitch - a.bw) % 8 != 0) ++w.pitch;
    const auto halo_bytes = [&](int pr) { return (((size_t)((pr - 1) * a.SY + a.KY) * w.pitch * a.IC + 1023) / 1024) * 1024; };
    const auto wbytes = [&](int nf) { return (size_t)w.nsteps * nf * 1024; };
    int nf = 0;
    for (int cand : {4, 2}) {
        if (nf_forced != 0 && cand != nf_forced) continue;
        if (cand == 4 && a.bc <= 32 && nf_forced == 0) continue;
        if (wbytes(cand) + halo_bytes(1) <= kPatchLdsCap) {
            nf = cand;
            break;
        }
    }
    if (nf == 0) return hipErrorNotSupported;
    const int64_t nimg = (int64_t)a.M / ((int64_t)a.bh * a.bw);
    w.nslices = (uint32_t)((a.bc + 16 * nf - 1) / (16 * nf));
    // Rows per patch. A patch of ngr fragment groups keeps ceil(ngr / 4) groups per SIMD busy one after the other, and a
    // workgroup walks tpg patches, each with a fixed cost (requests, re-bias, two barriers, epilogue tails): the rows
    // that minimise tpg * (ceil(ngr / 4) + 1/2), single-buffered patches of a multi-patch workgroup priced 15 % higher;
    // ties go to the taller patch (less halo).
    constexpr int cus = 256;  // MI355X
    int pr = 0;
    if (pr_forced > 0) {
        pr = std::min(pr_forced, a.bh);
        if (wbytes(nf) + halo_bytes(pr) > kPatchLdsCap) return hipErrorNotSupported;
    } else {
        double best = 0.0;
        for (int cand = 1; cand <= std::min(a.bh, 64); ++cand) {
            if (wbytes(nf) + halo_bytes(cand) > kPatchLdsCap) break;
            const int64_t np = nimg * ((a.bh + cand - 1) / cand);
            const int64_t groups = std::min<int64_t>(np, std::max<int64_t>(1, cus / (int64_t)w.nslices));
            const int64_t tpg = (np + groups - 1) / groups;
            const int64_t ngr = (((int64_t)cand * a.bw + 15) / 16 + npxf - 1) / npxf;
            double cost = (double)tpg * ((double)((ngr + 3) / 4) * (npxf / 4.0) + 0.5);
            if (tpg > 1 && wbytes(nf) + 2 * halo_bytes(cand) > kPatchLdsCap) cost *= 1.15;
            if (pr == 0 || cost <= best) {
                best = cost;
                pr = cand;
            }
        }
        if (pr == 0) return hipErrorNotSupported;
    }
    w.PR = pr;
    w.nrp = (a.bh + pr - 1) / pr;
    const int64_t np64 = nimg * w.nrp;
    if (np64 <= 0 || np64 > 0x7ffffff0LL) return hipErrorNotSupported;
    w.npatch = (uint32_t)np64;
    w.div_nrp = make_fastdiv((uint32_t)w.nrp);
    w.div_pitch = make_fastdiv((uint32_t)w.pitch);
    w.halo_bytes = (uint32_t)halo_bytes(pr);
    w.nblk = (int32_t)(w.halo_bytes / 1024);
    w.nbuf = wbytes(nf) + 2 * (size_t)w.halo_bytes <= kPatchLdsCap ? 2 : 1;
    const uint32_t want_groups = (uint32_t)std::max<int64_t>(1, cus / (int64_t)w.nslices);
    w.ngroups = std::min<uint32_t>(w.npatch, want_groups);
    w.tpg = (w.npatch + w.ngroups - 1) / w.ngroups;
    w.ngroups = (w.npatch + w.tpg - 1) / w.tpg;
    if (w.tpg == 1) w.nbuf = 1;
    if ((uint64_t)w.ngroups * w.nslices > 0x7ffffff0ull) return hipErrorNotSupported;
    // slot offsets and keys must stay small enough for 32-bit byte arithmetic inside the LDS (they do: the LDS is 160 KiB)
    const size_t lds = wbytes(nf) + (size_t)w.nbuf * w.halo_bytes;
#ifdef PATCH_TRACE
    w.trace = g_probe_trace;
#endif
    if (tls_launch.log != nullptr)
        tls_launch.log->add(3, "conv: patch kernel, %d channels per slice, %d rows per patch, %d patch buffer(s), %u workgroups of %d waves x %u patches, groups of %d fragment(s)",
                            16 * nf, w.PR, w.nbuf, w.ngroups * w.nslices, waves, w.tpg, npxf);
    if (nf == 4) return launch_patch_u<4>(w, lds, ulog, waves, npxf, stream);
    return launch_patch_u<2>(w, lds, ulog, waves, npxf, stream);
}

}  // namespace nce
