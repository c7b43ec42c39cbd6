// Pieces shared by the convolution kernels that compute 16x16x64 MFMA tiles with the channel permutation
// "lane (pixel c, quarter q) holds 4*NF consecutive channels": the fill line for out-of-image taps, the
// wave-uniform epilogue constants and the fused PPE epilogue + store.
#pragma once

#include "nce_conv_common.h"

namespace nce {
namespace wres_detail {

// One 64-byte line per byte value: lanes whose tap lies outside the image load the input zero point from
// here instead of the activation tensor, so every activation load is unconditional (nothing has to
// wait for it until the matrix instruction that consumes it).
struct FillTable {
    uint8_t b[256][64];
};
constexpr FillTable make_fill_table() {
    FillTable t{};
    for (int v = 0; v < 256; ++v)
        for (int i = 0; i < 64; ++i) t.b[v][i] = (uint8_t)v;
    return t;
}
// (not const: a constant-address-space pointer selected against a global one would turn every activation load
// into a FLAT load, which also counts against the LDS wait counter)
static __device__ FillTable g_fill = make_fill_table();

// Channel (within the slice) that row i of channel fragment f carries: lane (c, q) of the result then
// holds channels 4*NF*q .. 4*NF*q + 4*NF-1, consecutive, for f = 0..NF-1 and its 4 registers.
template <int NF>
__device__ __forceinline__ int channel_of_frag_row(int f, int i) {
    return 4 * NF * (i >> 2) + 4 * f + (i & 3);
}

// bits [lo, hi) of a 32-bit mask (empty when hi <= lo; hi - lo <= 32)
__device__ __forceinline__ uint32_t bit_range(int lo, int hi) {
    return hi > lo ? ((0xFFFFFFFFu >> (32 - (hi - lo))) << lo) : 0u;
}

// Wave-uniform constants of the FP64 epilogues. Outputs are computed as bytes 0..255: signed outputs 128
// higher, flipped back by an XOR on the packed word; truncating conversion to int32, one v_med3_i32, byte
// insert.
struct EpiPack {
    int32_t ilo, ihi;   // clamp bounds with the zero point (+128 for signed outputs) added: 0 <= ilo <= ihi <= 255
    uint32_t flip;      // 0x80808080 for signed outputs
    double zp_fold;     // what B carries on top of the bias term: the output zero point (+128 for signed outputs)
    double pcz;         // slope mode: rounding constant of the slope + zp_fold * (1 - slope)
    int32_t pmq;        // high-word slope mode: slope * 2^32 ...
    int64_t cpz;        // ... and (rounding constant + zp_fold * (1 - slope)) * 2^32
};

__device__ __forceinline__ EpiPack epi_pack_setup(const PpeF64& pu) {
    EpiPack e;
    const int32_t sb = pu.lo_zp < 0 ? 128 : 0;  // only signed storage clamps below zero
    e.ilo = pu.lo_zp + sb;
    e.ihi = pu.hi_zp + sb;
    e.flip = sb ? 0x80808080u : 0u;
    e.zp_fold = (double)(pu.zp + sb);
    e.pcz = pu.pc + e.zp_fold - e.zp_fold * pu.pm;  // exact: 8 integer bits, at most 31 fractional bits
    e.pmq = 0;
    e.cpz = 0;
    return e;
}

typedef unsigned short fz_u16x2 __attribute__((ext_vector_type(2)));

// (CA, FZP: ConvArgs and a pointer to FuseAdd, either of them possibly in the constant address space)
template <int NF, int BF, int PMODE, bool FZ = false, typename CA, typename FZP = const FuseAdd*>
__device__ __forceinline__ void wres_epilogue(const CA& a, const EpiSmem& s, const double* sBfull, const int32_t* sCorr,
                                              const v4i (&acc)[NF][BF], const int32_t (&dws)[BF], int q, int noc,
                                              uint8_t* const (&dst)[BF], const bool (&valid)[BF], const PpeF64& pu,
                                              const EpiPack& ep, FZP fz = nullptr, const uint4* other = nullptr) {
    const int ch0 = 4 * NF * q;
    if (ch0 >= noc) return;
    if constexpr (PMODE == PPE_MODE_INT && BF > 1) {
        // The 64-bit integer form runs one pixel fragment at a time: over all BF at once it needs more registers than the
        // reduction loops of its callers, and then the whole kernel spills (a reload from scratch memory is a vector
        // memory operation: the wait for it also waits for every activation load the kernel keeps in flight).
#pragma unroll
        for (int x = 0; x < BF; ++x) {
            v4i a1[NF][1];
#pragma unroll
            for (int f = 0; f < NF; ++f) a1[f][0] = acc[f][x];
            uint8_t* const d1[1] = {dst[x]};
            const bool v1[1] = {valid[x]};
            const int32_t w1[1] = {dws[x]};
            wres_epilogue<NF, 1, PPE_MODE_INT, FZ>(a, s, sBfull, sCorr, a1, w1, q, noc, d1, v1, pu, ep, fz, FZ ? other + x : other);
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }
    const PpeDev ppe_args = generic_copy<PpeDev>(a.ppe);
    static_assert(!FZ || NF == 4, "fused add: a lane holds 16 channels");
    uint32_t wo[BF][NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
#pragma unroll
        for (int x = 0; x < BF; ++x) wo[x][f] = 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int c = ch0 + 4 * f + r;
            double M = 0.0, B = 0.0;
            int32_t w2 = 0, bias = 0, corr = 0;
            // (the activation zero point is already in the wave's constants: da * sum of the channel's weights)
            int32_t mq = 0;
            int64_t cq = 0;
            if (PMODE == PPE_MODE_INT) {
                w2 = s.w2[c];
                bias = s.bias[c];
                corr = sCorr[c];
            } else if (PMODE == PPE_MODE_HI || PMODE == PPE_MODE_HI_SLOPE) {
                mq = sCorr[c];
                cq = reinterpret_cast<const int64_t*>(sBfull)[c];
            } else {
                M = s.M[c];
                B = sBfull[c];
            }
#pragma unroll
            for (int x = 0; x < BF; ++x) {
                const int32_t av = acc[f][x][r] + dws[x];  // (+ dw * sum of the pixel's activations; 0 when dw == 0)
                if (PMODE == PPE_MODE_INT) {
                    const int32_t y = ppe_apply((int32_t)((uint32_t)av + (uint32_t)corr), bias, table_mult(w2), table_shift(w2), ppe_args);
                    wo[x][f] |= ((uint32_t)y & 0xFFu) << (8 * r);
                } else if (PMODE == PPE_MODE_HI) {
                    // y = floor(((av + bias') * mult + 2^(shift-1) + zp * 2^shift) / 2^shift), everything scaled
                    // by 2^(32 - shift) so that the division is "take the high word": one 32 x 32 + 64 bit
                    // multiply-add per output. mq and cq are set up per wave (see kernel).
                    const int32_t y = clamp_med3((int32_t)(((int64_t)av * mq + cq) >> 32), ep.ilo, ep.ihi);
                    wo[x][f] = r == 0 ? (uint32_t)y : (wo[x][f] | ((uint32_t)y << (8 * r)));
                } else if (PMODE == PPE_MODE_HI_SLOPE) {
                    // The same with a negative slope |slope| <= 1: rz is the value before the slope (zero point
                    // added), nz the value after it, both exact; the larger of the two is the result (below
                    // zero the slope raises a value, from zero up it does not).
                    const int32_t rz = (int32_t)(((int64_t)av * mq + cq) >> 32);
                    const int32_t nz = (int32_t)(((int64_t)rz * ep.pmq + ep.cpz) >> 32);
                    const int32_t y = min(max(max(rz, nz), ep.ilo), ep.ihi);
                    wo[x][f] = r == 0 ? (uint32_t)y : (wo[x][f] | ((uint32_t)y << (8 * r)));
                } else if (PMODE == PPE_MODE_FOLDED) {
                    // The conversion truncates; below zero that differs from floor, but every value below
                    // zero (and floor's -1 for a value in (-1, 0)) clamps to ep.ilo >= 0 either way.
                    const int32_t y = clamp_med3((int32_t)__builtin_fma((double)av, M, B), ep.ilo, ep.ihi);
                    wo[x][f] = r == 0 ? (uint32_t)y : (wo[x][f] | ((uint32_t)y << (8 * r)));
                } else {
                    // Slope mode, everything shifted up by the output zero point zp (B carries it, as in folded
                    // mode): tz = t + zp. Below zero the slope applies to floor(t) = floor(tz) - zp, which
                    // ep.pcz folds in: n = floor(t) * pm + pc + zp, exact. Both candidates are converted by
                    // truncation - right for values >= 0, and below 0 everything clamps to ep.ilo >= 0.
                    const double tz = __builtin_fma((double)av, M, B);
                    const double n = __builtin_fma(__builtin_floor(tz), pu.pm, ep.pcz);
                    const int32_t y = clamp_med3(tz < ep.zp_fold ? (int32_t)n : (int32_t)tz, ep.ilo, ep.ihi);
                    wo[x][f] = r == 0 ? (uint32_t)y : (wo[x][f] | ((uint32_t)y << (8 * r)));
                }
            }
        }
        if (PMODE != PPE_MODE_INT) {
#pragma unroll
            for (int x = 0; x < BF; ++x) wo[x][f] ^= ep.flip;
        }
        __builtin_amdgcn_sched_barrier(0);  // one fragment's constants live at a time
    }
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        if (!valid[x]) continue;
        if constexpr (NF == 4) store_channels16(dst[x] + ch0 * a.out_sc, a.out_sc, wo[x][0], wo[x][1], wo[x][2], wo[x][3]);
        else store_channels8(dst[x] + ch0 * a.out_sc, a.out_sc, wo[x][0], wo[x][1]);
    }
    if constexpr (FZ) {
        // The add on the bytes just stored (a.out_sc == 1 here): byte i of both inputs as a pair of 16-bit values, one
        // 16-bit dot product with the two input multipliers, the high word of one multiply-add, clamp, byte insert.
#pragma unroll
        for (int x = 0; x < BF; ++x) {
            if (!valid[x]) continue;
            const uint32_t ob[4] = {other[x].x, other[x].y, other[x].z, other[x].w};
            uint32_t r[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t ua = wo[x][d] ^ fz->in_flip, ub = ob[d] ^ fz->in_flip;
                uint32_t packed = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t pair = __builtin_amdgcn_perm(ub, ua, 0x0c040c00u + (uint32_t)i * 0x00010001u);
                    const int32_t sum = (int32_t)__builtin_amdgcn_udot2(__builtin_bit_cast(fz_u16x2, pair), __builtin_bit_cast(fz_u16x2, fz->mults),
                                                                         (uint32_t)fz->c0h, false);
                    const int32_t y = clamp_med3((int32_t)(((int64_t)sum * fz->mq + fz->cq) >> 32), fz->ilo, fz->ihi);
                    packed = i == 0 ? (uint32_t)y : (packed | ((uint32_t)y << (8 * i)));
                }
                r[d] = packed ^ fz->flip;
            }
            *reinterpret_cast<uint4*>(fz->out + ((dst[x] + ch0) - a.out)) = make_uint4(r[0], r[1], r[2], r[3]);
        }
    }
}

}  // namespace wres_detail
}  // namespace nce
