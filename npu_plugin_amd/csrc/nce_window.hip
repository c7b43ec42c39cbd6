// DWCONV, AVEPOOL and MAXPOOL tasks: per-channel sliding-window ops on NHWC activations.
// Semantics (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc):
//   DWCONV  :834-945   acc = sum (a - zp_a) * (w - zp_w) over in-image taps, scale/bias from the table
//   AVEPOOL :1805-1905 acc = sum (a - zp_a) over in-image taps (window weight 1, :907-913), the
//                      1/(KY*KX) lives in the PPE scale
//   MAXPOOL :1759-1803 max of the raw values, scale 1 / shift 0 / zero point 0, clamp only
// Depthwise weights are one 16-byte-multiple row per channel holding the KY*KX taps row-major
// (src/vpux_compiler/src/dialect/VPU/utils/const_utils.cpp:101-120,216-243).
//
// Memory-bound kernels: a lane owns one 16-channel group (one 128-bit load per tap) of one output
// pixel; adjacent lanes own adjacent channel groups, so a wavefront reads whole NHWC pixels
// contiguously. Arithmetic is kept below the memory time:
//   * depthwise sums over a compile-time window (2x2, 3x3, 5x5) take two taps per instruction: v_perm_b32
//     pairs a byte of two taps as 16-bit values, v_dot2_i32_i16 multiplies them with the channel's weight
//     pair. Other sums run in FP32 on v_cvt_f32_ubyteN (byte -> float in one instruction) + v_fma_f32:
//     every partial sum is an integer below 2^24 (121 taps * 255 * 255), so FP32 is exact.
//   * bytes are taken as unsigned (i8 storage is re-biased by x ^ 0x80) and out-of-image taps are
//     filled with the zero point, so they contribute 0; the constant  -zp * sum(w)  is folded into
//     the per-channel bias. (Max pool keeps the clamped in-window pixel instead: the maximum is the same.)
//   * the requantize runs in FP64 (see nce_ppe_device.h); shifts above 52 take the integer path.
//   * MAXPOOL compares two channels per instruction (even / odd bytes as packed u16).
#include "nce_conv_common.h"

namespace nce {
namespace {

enum { MODE_DW = 0, MODE_AVG = 1, MODE_MAX = 2 };

constexpr int SLAB_GROUPS = 8;             // channel groups (of 16) one block works on
constexpr int SLAB_CH = SLAB_GROUPS * 16;  // 128 channels
constexpr int NT = 256;

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short s16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float ubyte_f32(uint32_t w, int i) {
    // the compiler turns this into v_cvt_f32_ubyte{i}
    return (float)((w >> (8 * i)) & 0xFFu);
}

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    const u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    const u16x2 r = __builtin_elementwise_min(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}

// FP64 requantize of 16 channel sums with per-channel constants, packed into 4 dwords.
template <int PMODE>
__device__ __forceinline__ void requant16(const float (&acc)[16], const double* M, const double* B, const PpeF64& pu,
                                          uint32_t (&wo)[4]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int32_t y = ppe_finish_mode<PMODE>(__builtin_fma((double)acc[i], M[i], B[i]), pu);
        const uint32_t b = (uint32_t)y & 0xFFu;
        wo[i >> 2] = (i & 3) == 0 ? b : (wo[i >> 2] | (b << (8 * (i & 3))));
    }
}

struct WinArgs {
    TaskDev t;
    Box box;
    int64_t npix;
    int32_t items_per_thread;
    uint32_t nblocks;  // item blocks per channel slab (the grid is padded to a multiple of the XCD count)
    uint32_t a_xor;   // 0x80808080 for i8 activations
    uint32_t fill;    // word of re-biased zero-point bytes for out-of-image taps
    int32_t zpu;      // zero point of the re-biased (unsigned) activation bytes
    // I32 kernels (item count and tensor strides below 2^31): divisors of the item decomposition
    int32_t nslab_full;            // channel groups of every slab but the last
    FastDiv div_full, div_last;    // by the channel groups of a full slab / of the last slab
    FastDiv div_bw, div_bh;
};

// KK = 2, 3, 5: KY == KX == KK known at compile time. All taps of an item are then requested before the first
// one is used - unconditionally, from coordinates clamped into the image, with out-of-image taps replaced
// afterwards - so that an item costs one memory round trip instead of one per tap. KK = 0: any window, taps
// loaded one after the other.
// I32: the item count and every tensor stride fit 31 bits. The decomposition of an item into channel group, column,
// row and image then runs on multiply-high divisions and index * stride is one 32 x 32 + 64 bit multiply-add;
// the general kernel pays three 64-bit divisions per item, which cost more than the window itself.
template <int MODE, int KK, bool I32>
__global__ __launch_bounds__(NT) void window_kernel(WinArgs a) {
    prefetch_kernel_arguments<sizeof(WinArgs)>();
    // MODE_DW: [tap][SLAB_CH] floats of (w - zp_w); then per-channel FP64 scale constants
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ double sM[SLAB_CH], sB[SLAB_CH];
    __shared__ int32_t sMult[SLAB_CH], sShift[SLAB_CH], sBias[SLAB_CH], sCorr[SLAB_CH];

    const TaskDev& t = a.t;
    const Box& box = a.box;
    const int32_t cgroups = box.bc >> 4;
    const int32_t slab0 = blockIdx.y * SLAB_GROUPS;
    const int32_t nslab = min(SLAB_GROUPS, cgroups - slab0);
    const int ntaps = t.ky * t.kx;
    float* s_w = reinterpret_cast<float*>(smem);

    // ---- per-channel constants ---------------------------------------------------------------
    // One channel per thread (a slab has at most SLAB_CH = 128 channels, the block 256 threads): the weight-table
    // row and the channel's weights are requested together, the workgroup then agrees on the PPE specialisation
    // it runs (uniform), and the constants for it are written - one memory round trip before the main loop.
    static_assert(NT >= SLAB_CH, "one channel per thread");
    const int ch = threadIdx.x;
    const bool has_ch = MODE != MODE_MAX && ch < nslab * 16;
    int32_t mult = t.ppe.quant_mult, shift = t.ppe.quant_shift, bias = 0, wsum = 0;
    if (has_ch) {
        const int32_t c = box.z0 + slab0 * 16 + ch;
        if (t.table != nullptr) {
            const int32_t* row = t.table + (int64_t)c * t.table_stride;
            mult = table_mult(row[2]);
            shift = table_shift(row[2]);
            bias = row[3];
        }
        if (MODE == MODE_DW) {
            const uint8_t* row = t.weights + (int64_t)c * t.w_stride_oc;
            if constexpr (KK > 0) {
                // compile-time windows: (w - zp_w) of taps 2j and 2j + 1 as a pair of 16-bit values, the operand of
                // v_dot2_i32_i16 (two taps of a channel per instruction)
                uint32_t* s_w2 = reinterpret_cast<uint32_t*>(smem);
                for (int j = 0; j < (KK * KK + 1) / 2; ++j) {
                    int32_t wv[2] = {0, 0};
                    for (int h = 0; h < 2; ++h) {
                        const int tap = 2 * j + h;
                        if (tap < KK * KK) wv[h] = (t.w_is_signed ? (int32_t)(int8_t)row[tap] : (int32_t)row[tap]) - t.w_zp;
                    }
                    wsum += wv[0] + wv[1];
                    s_w2[j * SLAB_CH + ch] = ((uint32_t)wv[0] & 0xFFFFu) | ((uint32_t)wv[1] << 16);
                }
            } else
            for (int tap = 0; tap < ntaps; ++tap) {
                const int32_t w = (t.w_is_signed ? (int32_t)(int8_t)row[tap] : (int32_t)row[tap]) - t.w_zp;
                wsum += w;
                s_w[tap * SLAB_CH + ch] = (float)w;
            }
        } else {
            wsum = ntaps;
        }
    }
    // (max pool has no scale: no constants, no workgroup synchronisation)
    bool use_int = false, may_sat = false;
    if constexpr (MODE != MODE_MAX) {
        const bool bad_shift = has_ch && shift > kMaxF64Shift;
        const bool small_shift = has_ch && ppe_may_saturate((int64_t)ntaps * (MODE == MODE_DW ? 65025 : 255), bias, mult, shift);
        // (one vote: bit 0 = a shift beyond FP64, bit 1 = possible int32 saturation)
        const int votes = __syncthreads_or((bad_shift ? 1 : 0) | (small_shift ? 2 : 0));
        use_int = (votes & 1) != 0;
        may_sat = (votes & 2) != 0;
    }
    const PpeF64 pu = ppe_f64_setup(t.ppe, may_sat);
    const int pmode = ppe_mode_of(pu, use_int);
    if (has_ch) {
        // out-of-image taps were filled with the zero point: remove zpu * sum(w) exactly
        const int32_t corr = -a.zpu * wsum;
        sMult[ch] = mult;
        sShift[ch] = shift;
        sBias[ch] = bias;
        sCorr[ch] = corr;  // |corr| < 2^23
        const double M = ppe_scale_M(mult, shift);
        sM[ch] = M;
        sB[ch] = ppe_mode_B(__builtin_fma((double)corr, M, ppe_scale_B(bias, M, shift, t.ppe.round_mode)), pmode, pu);
    }
    if constexpr (MODE != MODE_MAX) __syncthreads();

    const int64_t nitems = a.npix * nslab;
    const int64_t first = (int64_t)xcd_tile(blockIdx.x, a.nblocks) * NT * a.items_per_thread;
    for (int it = 0; it < a.items_per_thread; ++it) {
        const int64_t item = first + (int64_t)it * NT + threadIdx.x;
        if (item >= nitems) break;
        int32_t cg, bx, by;
        int64_t n;
        if constexpr (I32) {
            const uint32_t u = (uint32_t)item;
            const uint32_t r1 = fdiv(u, nslab == a.nslab_full ? a.div_full : a.div_last);
            cg = (int32_t)(u - r1 * (uint32_t)nslab);
            const uint32_t r2 = fdiv(r1, a.div_bw);
            bx = (int32_t)(r1 - r2 * (uint32_t)box.bw);
            const uint32_t r3 = fdiv(r2, a.div_bh);
            by = (int32_t)(r2 - r3 * (uint32_t)box.bh);
            n = r3;
        } else {
            cg = (int32_t)(item % nslab);
            int64_t r = item / nslab;
            bx = (int32_t)(r % box.bw);
            r /= box.bw;
            by = (int32_t)(r % box.bh);
            n = r / box.bh;
        }
        // index * stride
        auto mul = [](int32_t i, int64_t stride) { return I32 ? (int64_t)i * (int32_t)stride : (int64_t)i * stride; };
        const int32_t oc = box.z0 + ((slab0 + cg) << 4);
        const int32_t oy = box.y0 + by, ox = box.x0 + bx;
        const int32_t iy0 = oy * t.sy - t.pt, ix0 = ox * t.sx - t.pl;
        const uint8_t* src = t.in.data + mul((int32_t)n, t.in.sn) + oc;
        uint8_t* dst = t.out.data + mul((int32_t)n, t.out.sn) + mul(oy, t.out.sh) + mul(ox, t.out.sw) + oc * t.out.sc;

        if (MODE == MODE_MAX) {
            // even / odd bytes of each dword as packed u16; order-preserving re-bias for i8
            uint32_t me[4] = {0, 0, 0, 0}, mo[4] = {0, 0, 0, 0};
            if constexpr (KK > 0) {
                uint4 v[KK * KK];
#pragma unroll
                for (int ky = 0; ky < KK; ++ky)
#pragma unroll
                    for (int kx = 0; kx < KK; ++kx) {
                        const int32_t iy = min(max(iy0 + ky, 0), t.in.h - 1), ix = min(max(ix0 + kx, 0), t.in.w - 1);
                        v[ky * KK + kx] = *reinterpret_cast<const uint4*>(src + mul(iy, t.in.sh) + mul(ix, t.in.sw));
                    }
                if (a.a_xor != 0) {  // uniform: only i8 storage needs the order-preserving re-bias
#pragma unroll
                    for (int i = 0; i < KK * KK; ++i) v[i] = make_uint4(v[i].x ^ a.a_xor, v[i].y ^ a.a_xor, v[i].z ^ a.a_xor, v[i].w ^ a.a_xor);
                }
#pragma unroll
                for (int ky = 0; ky < KK; ++ky)
#pragma unroll
                    for (int kx = 0; kx < KK; ++kx) {
                        // (An out-of-image tap was loaded from its coordinates clamped into the image. Every window
                        // reaches into the image - the host sends other tasks to the general kernel -, so the clamped
                        // pixel is one of the window's own in-image pixels and the maximum is unchanged.)
                        const uint4 va = v[ky * KK + kx];
                        const uint32_t wa[4] = {va.x, va.y, va.z, va.w};
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            me[d] = pk_max_u16(me[d], wa[d] & 0x00FF00FFu);
                            mo[d] = pk_max_u16(mo[d], (wa[d] >> 8) & 0x00FF00FFu);
                        }
                    }
            } else
            for (int ky = 0; ky < t.ky; ++ky) {
                const int32_t iy = iy0 + ky;
                if ((uint32_t)iy >= (uint32_t)t.in.h) continue;
                for (int kx = 0; kx < t.kx; ++kx) {
                    const int32_t ix = ix0 + kx;
                    if ((uint32_t)ix >= (uint32_t)t.in.w) continue;
                    const uint4 va = *reinterpret_cast<const uint4*>(src + mul(iy, t.in.sh) + mul(ix, t.in.sw));
                    const uint32_t wa[4] = {va.x ^ a.a_xor, va.y ^ a.a_xor, va.z ^ a.a_xor, va.w ^ a.a_xor};
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        me[d] = pk_max_u16(me[d], wa[d] & 0x00FF00FFu);
                        mo[d] = pk_max_u16(mo[d], (wa[d] >> 8) & 0x00FF00FFu);
                    }
                }
            }
            // clamp in the re-biased domain (lo/hi shifted by 128 for i8), then undo the re-bias
            const uint32_t off = t.in.is_signed ? 128u : 0u;
            const uint32_t lo2 = ((uint32_t)(t.ppe.lo + (int32_t)off)) * 0x00010001u;
            const uint32_t hi2 = ((uint32_t)(t.ppe.hi + (int32_t)off)) * 0x00010001u;
            uint32_t wo[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t e = pk_min_u16(pk_max_u16(me[d], lo2), hi2);
                const uint32_t o = pk_min_u16(pk_max_u16(mo[d], lo2), hi2);
                wo[d] = (e | (o << 8)) ^ a.a_xor;
            }
            store_channels16(dst, t.out.sc, wo[0], wo[1], wo[2], wo[3]);
            continue;
        }

        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
        auto tap = [&](int ky, int kx, const uint4& va) {
                const uint32_t wa[4] = {va.x, va.y, va.z, va.w};
                if (MODE == MODE_DW) {
                    const float4* wp = reinterpret_cast<const float4*>(s_w + (ky * t.kx + kx) * SLAB_CH + (cg << 4));
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const float4 w4 = wp[d];
                        acc[4 * d + 0] = __builtin_fmaf(ubyte_f32(wa[d], 0), w4.x, acc[4 * d + 0]);
                        acc[4 * d + 1] = __builtin_fmaf(ubyte_f32(wa[d], 1), w4.y, acc[4 * d + 1]);
                        acc[4 * d + 2] = __builtin_fmaf(ubyte_f32(wa[d], 2), w4.z, acc[4 * d + 2]);
                        acc[4 * d + 3] = __builtin_fmaf(ubyte_f32(wa[d], 3), w4.w, acc[4 * d + 3]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[i] += ubyte_f32(wa[i >> 2], i & 3);
                }
        };
        if constexpr (KK > 0) {
            uint4 v[KK * KK];
#pragma unroll
            for (int ky = 0; ky < KK; ++ky)
#pragma unroll
                for (int kx = 0; kx < KK; ++kx) {
                    const int32_t iy = min(max(iy0 + ky, 0), t.in.h - 1), ix = min(max(ix0 + kx, 0), t.in.w - 1);
                    v[ky * KK + kx] = *reinterpret_cast<const uint4*>(src + mul(iy, t.in.sh) + mul(ix, t.in.sw));
                }
            // Out-of-image taps take the zero point. Most wavefronts hold no such tap: the replacement runs only where
            // one does (uniform branch).
            const bool inside = iy0 >= 0 && ix0 >= 0 && iy0 + KK <= t.in.h && ix0 + KK <= t.in.w;
            if (a.a_xor != 0) {  // uniform: i8 storage is re-biased to unsigned bytes
#pragma unroll
                for (int i = 0; i < KK * KK; ++i) v[i] = make_uint4(v[i].x ^ a.a_xor, v[i].y ^ a.a_xor, v[i].z ^ a.a_xor, v[i].w ^ a.a_xor);
            }
            if (!__all(inside)) {
                const uint32_t fr = a.fill;
#pragma unroll
                for (int ky = 0; ky < KK; ++ky)
#pragma unroll
                    for (int kx = 0; kx < KK; ++kx) {
                        const bool ok = (uint32_t)(iy0 + ky) < (uint32_t)t.in.h && (uint32_t)(ix0 + kx) < (uint32_t)t.in.w;
                        uint4& r = v[ky * KK + kx];
                        r = make_uint4(ok ? r.x : fr, ok ? r.y : fr, ok ? r.z : fr, ok ? r.w : fr);
                    }
            }
            auto fixed = [&](int ky, int kx) { return v[ky * KK + kx]; };  // re-biased bytes of a tap
            if constexpr (MODE == MODE_DW) {
                // Two taps per instruction: v_perm_b32 pairs byte i of both taps as 16-bit values, v_dot2_i32_i16
                // multiplies the pair with the channel's weight pair and accumulates (exact, int32).
                int32_t acci[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) acci[i] = 0;
                const uint32_t* wp2 = reinterpret_cast<const uint32_t*>(smem) + (cg << 4);
#pragma unroll
                for (int j = 0; j < (KK * KK + 1) / 2; ++j) {
                    const uint4 ra = fixed((2 * j) / KK, (2 * j) % KK);
                    const uint4 rb = 2 * j + 1 < KK * KK ? fixed((2 * j + 1) / KK, (2 * j + 1) % KK) : make_uint4(0, 0, 0, 0);
                    const uint32_t wa[4] = {ra.x, ra.y, ra.z, ra.w}, wb[4] = {rb.x, rb.y, rb.z, rb.w};
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint4 w4 = *reinterpret_cast<const uint4*>(wp2 + j * SLAB_CH + 4 * d);
                        const uint32_t wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t pair = __builtin_amdgcn_perm(wb[d], wa[d], 0x0c040c00u + (uint32_t)i * 0x00010001u);
                            acci[4 * d + i] = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2, pair), __builtin_bit_cast(s16x2, wv[i]),
                                                                     acci[4 * d + i], false);
                        }
                    }
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = (float)acci[i];  // exact: below 2^24
            } else {
#pragma unroll
                for (int ky = 0; ky < KK; ++ky)
#pragma unroll
                    for (int kx = 0; kx < KK; ++kx) tap(ky, kx, fixed(ky, kx));
            }
        } else {
            for (int ky = 0; ky < t.ky; ++ky) {
                const int32_t iy = iy0 + ky;
                const bool row_in = (uint32_t)iy < (uint32_t)t.in.h;
                for (int kx = 0; kx < t.kx; ++kx) {
                    const int32_t ix = ix0 + kx;
                    uint4 va = make_uint4(a.fill, a.fill, a.fill, a.fill);
                    if (row_in && (uint32_t)ix < (uint32_t)t.in.w) {
                        va = *reinterpret_cast<const uint4*>(src + mul(iy, t.in.sh) + mul(ix, t.in.sw));
                        va.x ^= a.a_xor;
                        va.y ^= a.a_xor;
                        va.z ^= a.a_xor;
                        va.w ^= a.a_xor;
                    }
                    tap(ky, kx, va);
                }
            }
        }

        uint32_t wo[4];
        const int chl = cg << 4;
        if (pmode == PPE_MODE_FOLDED) requant16<PPE_MODE_FOLDED>(acc, sM + chl, sB + chl, pu, wo);
        else if (pmode == PPE_MODE_SLOPE) requant16<PPE_MODE_SLOPE>(acc, sM + chl, sB + chl, pu, wo);
        else {
            wo[0] = wo[1] = wo[2] = wo[3] = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                // acc + corr is the true accumulator (|.| < 2^23); the table bias is added in 64 bits inside
                const int32_t y = ppe_apply((int32_t)acc[i] + sCorr[chl + i], sBias[chl + i], sMult[chl + i], sShift[chl + i], t.ppe);
                wo[i >> 2] |= ((uint32_t)y & 0xFFu) << (8 * (i & 3));
            }
        }
        store_channels16(dst, t.out.sc, wo[0], wo[1], wo[2], wo[3]);
    }
}

template <int MODE, int KK, bool I32>
hipError_t launch_window_i32(const WinArgs& a, int64_t blocks, int nslabs, size_t lds, hipStream_t s) {
    static LdsGrant grant;  // large depthwise kernels: opt in to more than the default dynamic LDS
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(&window_kernel<MODE, KK, I32>), lds, 32 * 1024); e != hipSuccess) return e;
    return emit(window_kernel<MODE, KK, I32>, dim3(xcd_grid((unsigned)blocks), (unsigned)nslabs), dim3(NT), lds, s, a);
}

template <int MODE, int KK>
hipError_t launch_window_kk(const TaskDev& t, const Box& box, hipStream_t s) {
    WinArgs a;
    a.t = t;
    a.box = box;
    a.npix = (int64_t)t.out.n * box.bh * box.bw;
    const int32_t cgroups = box.bc >> 4;
    if (a.npix == 0 || cgroups == 0) return hipSuccess;
    const int nslabs = (cgroups + SLAB_GROUPS - 1) / SLAB_GROUPS;
    const int64_t items = a.npix * (cgroups < SLAB_GROUPS ? cgroups : SLAB_GROUPS);
    // (several items per thread amortise the per-workgroup constants of large tasks; max pool has none and measured
    // fastest with one item per thread at every size)
    a.items_per_thread = (MODE != MODE_MAX && items > (int64_t)NT * 8192) ? 4 : 1;
    const int64_t blocks = (items + NT * a.items_per_thread - 1) / (NT * a.items_per_thread);
    if (blocks > 0x7ffffff0LL) return hipErrorInvalidValue;
    a.nblocks = (uint32_t)blocks;
    a.a_xor = t.in.is_signed ? 0x80808080u : 0u;
    a.zpu = t.in.zp + (t.in.is_signed ? 128 : 0);
    a.fill = (uint32_t)a.zpu * 0x01010101u;
    const size_t lds = MODE == MODE_DW ? (size_t)t.ky * t.kx * SLAB_CH * sizeof(float) : 0;
    const int32_t full = cgroups < SLAB_GROUPS ? cgroups : SLAB_GROUPS;
    a.nslab_full = full;
    a.div_full = make_fastdiv((uint32_t)full);
    a.div_last = make_fastdiv((uint32_t)(cgroups - (nslabs - 1) * SLAB_GROUPS));
    a.div_bw = make_fastdiv((uint32_t)box.bw);
    a.div_bh = make_fastdiv((uint32_t)box.bh);
    bool i32 = blocks * NT * a.items_per_thread < 0x7fffffffLL;
    for (const int64_t st : {t.in.sn, t.in.sh, t.in.sw, t.out.sn, t.out.sh, t.out.sw}) i32 = i32 && st >= 0 && st <= 0x7fffffffLL;
    if (i32) return launch_window_i32<MODE, KK, true>(a, blocks, nslabs, lds, s);
    return launch_window_i32<MODE, KK, false>(a, blocks, nslabs, lds, s);
}

template <int MODE>
hipError_t launch_window(const TaskDev& t, const Box& box, hipStream_t s) {
    if (MODE == MODE_MAX) {
        // the compile-time windows of the max pool rely on every window of the box overlapping the image
        const bool reach = t.pt < t.ky && t.pl < t.kx && (int64_t)(box.y0 + box.bh - 1) * t.sy - t.pt <= t.in.h - 1 &&
                           (int64_t)(box.x0 + box.bw - 1) * t.sx - t.pl <= t.in.w - 1;
        if (!reach) return launch_window_kk<MODE, 0>(t, box, s);
    }
    if (t.ky == 3 && t.kx == 3) return launch_window_kk<MODE, 3>(t, box, s);
    if (t.ky == 2 && t.kx == 2) return launch_window_kk<MODE, 2>(t, box, s);
    if (t.ky == 5 && t.kx == 5) return launch_window_kk<MODE, 5>(t, box, s);
    return launch_window_kk<MODE, 0>(t, box, s);
}

}  // namespace

hipError_t launch_pool(const TaskDev& t, const Box& box, bool is_max, hipStream_t stream) {
    return is_max ? launch_window<MODE_MAX>(t, box, stream) : launch_window<MODE_AVG>(t, box, stream);
}

hipError_t launch_dwconv(const TaskDev& t, const Box& box, hipStream_t stream) {
    return launch_window<MODE_DW>(t, box, stream);
}

}  // namespace nce
