// CONV task, weights-resident implicit GEMM on v_mfma_i32_16x16x64_i8.
//
// A workgroup owns one slice of 16*NF output channels and a run of pixel tiles. It stages the WHOLE
// reduction (KY*KX*IC bytes) of its channels in LDS once, as 1 KiB blocks that one ds_read_b128 per lane turns
// into an MFMA operand, and after that single barrier its wavefronts never synchronise again: each wave walks its own tiles of 16*BF output
// pixels, loads the activation operand straight from global memory and runs the fused PPE on its
// accumulators.
//
// Why 16x16x64: the B operand of that instruction is 16 pixels x 64 reduction bytes with lane
// (c = lane % 16, q = lane / 16) holding bytes 16q..16q+15 of pixel c. For NHWC activations those are
// the four 16-byte quarters of one pixel's 64 consecutive channels, and the result layout (lane holds
// rows 4q..4q+3 of column c) lets the four lanes of a pixel store 64 consecutive output bytes.
//
// Lane order of memory instructions matters more than the bytes they move: a global load whose four
// neighbouring lanes read one 64-byte run costs the texture addresser a quarter of one whose runs are
// spread over four quads of lanes, and an LDS access whose lanes share a bank group is serialised. Hence both
// operands are fetched with lane 4*row + piece: the weights are stored to LDS as fetched (row-major blocks whose
// pieces are permuted so that the operand reads are conflict-free, nce_conv_lds.h), the activations (template flag
// TRL, when pixels are more than 64 bytes apart) are moved into operand order (lane 16*piece + row) with
// ds_bpermute_b32.
//
// The reduction is cut in steps of 64 bytes = four 16-byte units; unit u covers bytes 16u..16u+15 of
// the OYXI weight row, i.e. tap u / (IC/16), input channels 16 * (u % (IC/16)). With IC a multiple of
// 64 a step never straddles taps and the tap bookkeeping is scalar; other channel counts take the
// per-lane path (template MODE 2). Semantics and the fused PPE are the ones of nce_conv.hip.
#include "nce_conv_epi.h"
#include "nce_conv_lds.h"
#include "nce_conv_pk.h"

#include <mutex>
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace nce {

struct WresArgs {
    ConvArgs a;
    int32_t k16;        // 16-byte units along the reduction
    int32_t nsteps;     // 64-byte steps (k16 rounded up to 4), padded to a multiple of the load depth
    int32_t ntaps;      // KY * KX
    int32_t nc64;       // 64-byte chunks along IC (fast path)
    uint32_t ntiles;    // pixel tiles of 16*BF pixels
    uint32_t ngroups;   // workgroups along pixels
    int32_t tpg;        // tiles per workgroup
    int32_t linear;     // 1x1, stride 1, no padding, whole dense tensors: pixel p sits at p * pixel stride
    int32_t cs;         // chunked kernel: reduction steps staged at a time
    FastDiv div_icg;    // by IC / 16
    FastDiv div_kx;     // by KX
    FastDiv div_nc64;   // by nc64
    int64_t row_adv;    // input offset from the last tap of a kernel row to the first of the next: in_sh - KX * in_sw
    // The tensor strides once more as 32-bit values (the host checks that they fit): index * stride is then one
    // 32 x 32 + 64 bit multiply-add instead of a 64-bit multiplication.
    int32_t in_sn32, in_sh32, in_sw32, out_sn32, out_sh32, out_sw32;
    FuseAdd fz;         // kernels with LM_PLAIN_FZ only
    int32_t fused;      // host: the launch must carry the add in fz (or fail with hipErrorNotSupported)
#ifdef WRES_TRACE
    uint64_t* trace;    // probe builds only: [workgroup < 256][wave < 8][8] timestamps (100 MHz) of this launch
#endif
};

#ifdef WRES_TRACE
#define WRES_MARK(i)                                                                                                       \
    do {                                                                                                                   \
        if (w.trace != nullptr && lane == 0 && blockIdx.x < 256)                                                           \
            w.trace[((size_t)blockIdx.x * 8 + wave) * 8 + (i)] = __builtin_amdgcn_s_memrealtime();                          \
    } while (0)
#else
#define WRES_MARK(i) do { } while (0)
#endif

// This file is compiled four times (the instantiations of one pass take about a minute): WRES_PART 0 holds the dispatcher,
// the 32-channel kernels and the chunked kernel, WRES_PART 1 the 64-channel kernels with 16- and 32-pixel tiles behind this
// entry point, WRES_PART 2 those with 64-pixel tiles, WRES_PART 3 the persistent form (nce_conv_pk.h).
#ifndef WRES_PART
#define WRES_PART 0
#endif
// Weight loads a lane keeps in flight while a slice is staged. Eight for the persistent form, whose layers stage while other
// workgroups of the XCD still compute (measured on the ResNet-50 graph at batch 32: 639 against 648 us); for separate launches
// eight is level with four (-0.4 % at batch 32 and 64, +1.4 % at batch 8) and sixteen slower (+2 %: registers).
#ifndef NCE_WB
#if WRES_PART == 3
#define NCE_WB 8
#else
#define NCE_WB 4
#endif
#endif
hipError_t launch_wres_nf4(WresArgs& w, int bf, int mode, int nwaves, int tpw, hipStream_t stream);
#ifdef WRES_TRACE
extern uint64_t* g_wres_trace;  // probe builds: 64 launch records, written round robin
extern uint32_t g_wres_trace_seq;
#endif

namespace {

using namespace wres_detail;

enum { WRES_FAST = 0, WRES_FAST_MASK = 1, WRES_GENERIC = 2 };

// Per reduction step (modes 0 and 1): input byte offset of the step's tap and channel chunk relative to the
// pixel's first tap, and the tap's bit in the per-pixel validity mask (0 for a padding step).
struct __attribute__((aligned(16))) StepEntry {
    int32_t off_lo, off_hi;
    uint32_t tap_bit;
    int32_t pad;
};
constexpr int kMaxSteps = 80;  // 144 KiB / (2 fragments * 1 KiB) = 72 steps, padded to the load depth

// D: reduction steps whose activation loads are in flight per wave; the host picks a D that divides the step
// count where it can and pads the step count otherwise (a padding step multiplies zero weights).
// TRL: transpose the activation operand after loading. The matrix instruction wants lane 16k + p to hold
// 16-byte piece k of pixel p, which as a load pattern sends the four pieces of a pixel from four
// different quads of lanes; the texture addresser then works on 64 separate pieces per instruction. When
// pixels are more than 64 bytes apart that can halve the speed of the whole reduction loop, so there the
// loads run with lane 4p + k (a pixel's 64 bytes from four neighbouring lanes) and ds_bpermute moves the
// registers into operand order. With IC == 64 the plain pattern already covers whole lines and is faster.
// TBL: read each step's input offset and tap bit from a table in LDS instead of walking the taps with scalar
// counters (pays when every step changes tap: kernels larger than 1x1 over 64 input channels).
// ASUM: weights whose zero point differs from their storage offset by dw. The product then carries the extra
// terms dw * (sum of the pixel's activation operand) + K * da * dw: the sum comes out of the matrix unit (one
// instruction per step and pixel fragment against an all-ones operand, every row of the result is the sum),
// the constant joins the per-channel constants.
// LM packs the three flags: 0 plain, 1 TRL, 2 TBL, 3 plain + ASUM, 4 TRL + ASUM.
enum { LM_PLAIN = 0, LM_TRL = 1, LM_TBL = 2, LM_PLAIN_ASUM = 3, LM_TRL_ASUM = 4, LM_PLAIN_FZ = 5 };  // 5: plain + fused residual add
// The workgroup's LDS tables besides the staged weights.
template <int OCT, int NSTEP>
struct WresSmem {
    int32_t sW2[OCT], sBias[OCT];
    double sM[OCT], sBc[OCT], sMd[OCT];  // scale, bias term, scale * da
    // Weight sums: every wave leaves the partial sums of the fragments it staged in its row of sWpart; after
    // the barrier every wave folds the total into its OWN copy of the per-channel constants, so that no
    // second barrier is needed.
    int32_t sWpart[8][OCT];
    int32_t sCorr[8][OCT];   // integer path: da * sum of weights
    double sBfull[8][OCT];   // FP64 paths: bias term + da * M * sum of weights (+ output zero point)
    int32_t sFlags;
    StepEntry sStep[NSTEP];  // per-lane mode: one entry per 16-byte unit
};
template <int NF, int MODE>
using WresSmemOf = WresSmem<16 * NF, MODE == WRES_GENERIC ? 4 * kMaxSteps : kMaxSteps>;

// No-op hook of the plain kernel (see conv_wres_body).
struct NoInputWait {
    __device__ __forceinline__ void operator()() const {}
};

// The work of one workgroup: pixel group `group` (of w.ngroups) of channel slice `slice`. sWt: the dynamic LDS for the
// weights; sm: the tables. input_wait() is called by every wave, in uniform control flow, after the first weight requests
// and before the first access to the input tensor: the persistent form of the kernel waits there for the layer that
// produces the input (it may synchronise the workgroup).
// WArgs: WresArgs, possibly qualified with the constant address space (the persistent form reads its arguments from a table
// in memory; through that address space the compiler treats them as it treats kernel arguments - unchanging, fetched
// where they are used).
template <int NF, int BF, int MODE, int D, int LM, typename WArgs, typename InputWait>
__device__ __forceinline__ void conv_wres_body(const WArgs& w, const uint32_t group, const uint32_t slice, uint8_t* const sWt,
                                               WresSmemOf<NF, MODE>& sm, const InputWait& input_wait) {
    constexpr bool TRL = LM == LM_TRL || LM == LM_TRL_ASUM;
    constexpr bool TBL = LM == LM_TBL;
    constexpr bool ASUM = LM == LM_PLAIN_ASUM || LM == LM_TRL_ASUM;
    constexpr bool FZ = LM == LM_PLAIN_FZ;
    constexpr int OCT = 16 * NF;
    constexpr int BP = 16 * BF;
    static_assert(NF == 2 || NF == 4, "channel fragments");
    static_assert(D >= 2 || !TRL, "the permute of the next step needs a second ring slot");
    static_assert(!(TRL && TBL) && !(TBL && MODE == WRES_GENERIC), "the step table serves the plain load order of modes 0 and 1");
    const auto& a = w.a;
    const PpeDev ppe_args = generic_copy<PpeDev>(a.ppe);  // (for the helpers that take a reference)

    auto& sW2 = sm.sW2;
    auto& sBias = sm.sBias;
    auto& sM = sm.sM;
    auto& sBc = sm.sBc;
    auto& sMd = sm.sMd;
    auto& sWpart = sm.sWpart;
    auto& sCorr = sm.sCorr;
    auto& sBfull = sm.sBfull;
    auto& sFlags = sm.sFlags;
    auto& sStep = sm.sStep;
    const EpiSmem es = {sM, sBc, sW2, sBias, nullptr, nullptr};

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: keeps the tile walk in scalar registers
    const int nwaves = blockDim.x >> 6;
    const int c16 = lane & 15;                  // pixel of a fragment this lane holds in matrix layout
    // Pixel-major lane order: lane 4p + j carries 16-byte piece j ^ 2*(p >> 3) of pixel (or weight row) p. The four
    // lanes of a pixel still cover its 64 bytes; the swap of the piece pairs for p >= 8 makes the 32 source lanes that
    // each half of the wave reads in the permute distinct modulo 32 (without it they collide in pairs).
    const int kswz = (lane & 3) ^ ((lane >> 4) & 2);
    const int pl = TRL ? lane >> 2 : c16;       // pixel and 16-byte piece this lane loads
    const int kc = TRL ? kswz : lane >> 4;
    const int to_mfma = 4 * (4 * c16 + ((lane >> 4) ^ (2 * (c16 >> 3))));  // ds_bpermute source of lane 16k + p: piece k of pixel p

    const int32_t oc0 = a.z0 + (int32_t)slice * OCT;
    const int32_t noc = min(OCT, a.z0 + a.bc - oc0);

    const int axor = (int)a.a_xor;
    const uint8_t* const fillp = &g_fill.b[(a.fill ^ a.a_xor) & 0xFFu][kc * 16];
    const int S = w.nsteps;
    const uint32_t t_end = min((group + 1) * (uint32_t)w.tpg, w.ntiles);
    uint32_t t = group * (uint32_t)w.tpg + wave;

    // state of the tile in flight
    const uint8_t* pbase[BF];
    uint8_t* dst[BF];
    bool valid[BF];
    uint32_t mask0[BF], mask1[BF];  // FAST_MASK: tap bits; GENERIC: row bits, column bits
    int32_t ls = 0;  // reduction step the next load belongs to
    // scalar iterator of the kernels that do not read the step table: (tap, chunk) and input offset of the next load
    int32_t it_kx = 0, it_c64 = 0, it_tap = 0;
    int64_t it_off = 0, tap_off = 0;
    v4i fb[D][BF];

    auto setup = [&]() {
#pragma unroll
        for (int x = 0; x < BF; ++x) {
            // (unsigned: a tile index past the end - a wave without a tile - may put the pixel index above 2^31)
            const uint32_t p = t * BP + 16 * x + pl;
            valid[x] = p < (uint32_t)a.M;
            const int32_t pc = valid[x] ? (int32_t)p : a.M - 1;  // lanes past the end compute a duplicate
            if (w.linear) {  // uniform: no decomposition into image, row and column
                const uint32_t ps = t * BP + 16 * x + c16;  // pixel this lane holds in matrix layout
                pbase[x] = a.in + (int64_t)pc * w.in_sw32 + (MODE == WRES_GENERIC ? 0 : kc * 16);
                valid[x] = ps < (uint32_t)a.M;
                dst[x] = a.out + (int64_t)(valid[x] ? (int32_t)ps : a.M - 1) * w.out_sw32 + oc0 * a.out_sc;
                mask0[x] = mask1[x] = 1;
                continue;
            }
            const int32_t rr = fdiv(pc, a.div_bw);
            const int32_t bx = pc - rr * a.bw;
            const int32_t n = fdiv(rr, a.div_bh);
            const int32_t by = rr - n * a.bh;
            const int32_t iy0 = (a.y0 + by) * a.SY - a.PT;
            const int32_t ix0 = (a.x0 + bx) * a.SX - a.PL;
            pbase[x] = a.in + (int64_t)n * w.in_sn32 + (int64_t)iy0 * w.in_sh32 + (int64_t)ix0 * w.in_sw32 + (MODE == WRES_GENERIC ? 0 : kc * 16);
            dst[x] = a.out + (int64_t)n * w.out_sn32 + (int64_t)(a.y0 + by) * w.out_sh32 + (int64_t)(a.x0 + bx) * w.out_sw32 + oc0 * a.out_sc;
            if (TRL) {  // results come out in matrix layout: take the address of pixel c16 from a lane that computed it
                const uint64_t dl = reinterpret_cast<uint64_t>(dst[x]);
                const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(16 * c16, (int)(uint32_t)dl);
                const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(16 * c16, (int)(uint32_t)(dl >> 32));
                dst[x] = reinterpret_cast<uint8_t*>(((uint64_t)hi << 32) | lo);
                valid[x] = t * BP + 16 * x + c16 < (uint32_t)a.M;
            }
            mask0[x] = mask1[x] = 0;
            if (MODE != WRES_FAST) {
                const uint32_t rows = bit_range(max(0, -iy0), min(a.KY, a.H - iy0));
                const uint32_t cols = bit_range(max(0, -ix0), min(a.KX, a.W - ix0));
                if (MODE == WRES_GENERIC) {
                    mask0[x] = rows;
                    mask1[x] = cols;
                } else {
                    uint32_t m = 0;
                    for (int ky = a.KY - 1; ky >= 0; --ky) m = (m << a.KX) | (((rows >> ky) & 1u) ? cols : 0u);
                    mask0[x] = m;
                }
            }
        }
        ls = 0;
        it_kx = it_c64 = it_tap = 0;
        it_off = tap_off = 0;
    };
    // Entry of reduction step st of the table described at StepEntry.
    auto step_entry = [&](int st) {
        const int tap = fdiv(st, w.div_nc64);
        const int c64 = st - tap * w.nc64;
        const int ky = fdiv(tap, w.div_kx);
        const int kx = tap - ky * a.KX;
        const bool real = tap < w.ntaps;  // padding steps stay on a readable address, their tap bit is clear
        const int64_t off = real ? (int64_t)ky * w.in_sh32 + (int64_t)kx * w.in_sw32 + c64 * 64 : 0;
        StepEntry e;
        e.off_lo = (int32_t)(uint32_t)off;
        e.off_hi = (int32_t)(off >> 32);
        e.tap_bit = real ? 1u << tap : 0u;
        e.pad = 0;
        return e;
    };
    // Per-lane mode: entry of 16-byte unit u of the reduction - input offset, bit of its kernel row (tap_bit)
    // and of its kernel column (pad). Units past the reduction's end have no bits: they read the fill value.
    auto unit_entry = [&](int u) {
        const int tap = fdiv(u, w.div_icg);
        const int icg = u - tap * a.ICG;
        const int ky = fdiv(tap, w.div_kx);
        const int kx = tap - ky * a.KX;
        const bool real = u < w.k16;
        const int64_t off = real ? (int64_t)ky * w.in_sh32 + (int64_t)kx * w.in_sw32 + icg * 16 : 0;
        StepEntry e;
        e.off_lo = (int32_t)(uint32_t)off;
        e.off_hi = (int32_t)(off >> 32);
        e.tap_bit = real ? 1u << ky : 0u;
        e.pad = real ? 1u << kx : 0u;
        return e;
    };
    // Request the activation operand of the next step for every pixel fragment (raw bytes). The table of
    // steps is valid after the workgroup's barrier; the first tile's first requests go out before it and
    // compute their entries (from_table = false).
    auto load_b = [&](v4i (&d)[BF], bool from_table = true) {
        if (MODE == WRES_GENERIC) {
            const int u = 4 * ls + kc;
            const StepEntry e = from_table ? sStep[u] : unit_entry(u);
            const int64_t off = ((int64_t)e.off_hi << 32) | (uint32_t)e.off_lo;
#pragma unroll
            for (int x = 0; x < BF; ++x) {
                const bool ok = (mask0[x] & e.tap_bit) != 0 && (mask1[x] & e.pad) != 0;
                const uint8_t* src = ok ? pbase[x] + off : fillp;
                d[x] = *reinterpret_cast<const v4i*>(src);
            }
            ++ls;
        } else if constexpr (!TBL) {
            // Scalar counters walk the taps. Additions only - the scalar unit has no cheap 64-bit multiply.
#pragma unroll
            for (int x = 0; x < BF; ++x) {
                const uint8_t* src = pbase[x] + it_off;
                if (MODE == WRES_FAST_MASK) src = ((mask0[x] >> it_tap) & 1u) ? src : fillp;
                d[x] = *reinterpret_cast<const v4i*>(src);
            }
            it_off += 64;
            if (++it_c64 == w.nc64) {
                it_c64 = 0;
                ++it_tap;
                tap_off += a.in_sw;
                if (++it_kx == a.KX) {
                    it_kx = 0;
                    tap_off += w.row_adv;
                }
                it_off = tap_off;
                if (it_tap >= w.ntaps) {  // padding steps: stay on a readable address
                    it_off = 0;
                    it_tap = 31;
                }
            }
        } else {
            // Input offset and tap bit of the step come from the table built once per workgroup: one LDS
            // read instead of a chain of scalar counters, compares and selects per step. (Not for the kernels
            // with permuted loads, whose LDS pipe is busy with operand reads and permutes, nor for 1x1 kernels,
            // which never change tap: measured slower there.)
            const StepEntry e = from_table ? sStep[ls] : step_entry(ls);
            const int64_t off = ((int64_t)e.off_hi << 32) | (uint32_t)e.off_lo;
#pragma unroll
            for (int x = 0; x < BF; ++x) {
                const uint8_t* src = pbase[x] + off;
                if (MODE == WRES_FAST_MASK) src = (mask0[x] & e.tap_bit) ? src : fillp;
                d[x] = *reinterpret_cast<const v4i*>(src);
            }
            ++ls;
        }
    };
    auto first_loads = [&](bool from_table) {
#pragma unroll
        for (int j = 0; j < D; ++j) load_b(fb[j], from_table);
    };
    // ---- stage the channel slice's weights in operand order; per-channel constants ---------------
    // The slice is S * NF blocks of 1 KiB: (step, channel fragment) -> 16 rows x 64 bytes, kept row-major with the four
    // 16-byte pieces of a row permuted (nce_conv_lds.h). A wave fetches a block with the four lanes 4i .. 4i + 3 on the
    // pieces of row i (a row's 64 bytes from four neighbouring lanes, each lane on the piece that belongs at ITS position)
    // and writes it where it stands: one linear, bank-conflict-free store, no lane exchange.
    {
        const int li = lane >> 2;
        const int64_t acc_bound = min((int64_t)a.ktot * 65025, (int64_t)2147483648LL);
        // The last wave also derives the per-channel PPE constants (lane = channel) while its weight
        // loads are in flight.
        const bool consts_wave = wave == nwaves - 1;
        int32_t tw2 = 0, tbias = 0;
        if (consts_wave && lane < noc) {
            const int32_t* trow = a.table + (int64_t)(oc0 + lane) * a.table_stride;
            tw2 = trow[2];
            tbias = trow[3];
        }
        auto do_consts = [&]() {
            const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
            const bool bad = lane < OCT && shift > kMaxF64Shift;
            const bool sat = lane < OCT && ppe_may_saturate(acc_bound, tbias, mult, shift);
            // High-word integer epilogue: needs mult * 2^(32 - shift) in int32 and the 64-bit constant (bias and
            // weight-sum terms, below 2^32 together, times the scale; rounding and zero-point terms) below 2^62.
            bool hi_bad = false;
            if (lane < noc) {
                hi_bad = shift < 1 || shift > 32 || ((int64_t)mult << (32 - min(shift, 32))) > 0x7fffffffLL;
                const double cb = ((__builtin_fabs((double)tbias) + 4294967296.0) * (double)mult + 2147483648.0 + 384.0 * __builtin_ldexp(1.0, shift));
                hi_bad = hi_bad || __builtin_ldexp(cb, 32 - shift) >= 4611686018427387904.0;
            }
            const int wf = (__any(bad) ? 1 : 0) | (__any(sat) ? 2 : 0) | (__any(hi_bad) ? 4 : 0);
            if (lane == 0) sFlags = wf;
            if (lane < OCT) {
                const double M = ppe_scale_M(mult, shift);
                const double B = ppe_scale_B(tbias, M, shift, a.ppe.round_mode);
                sW2[lane] = tw2;
                sBias[lane] = tbias;
                sM[lane] = M;
                sMd[lane] = M * (double)a.da;
                sBc[lane] = B;
            }
        };
        // Reduction step st, channel fragment f is one 1 KiB block of 16 rows (channels) x 64 bytes, kept row-major: lane
        // 4 r + j fetches the 16-byte piece that belongs at position j of row r (nce_conv_lds.h: the pieces of a row are
        // permuted so that the operand reads of the reduction loop touch every bank group once per clock), and writes it
        // where it stands - one linear, conflict-free store per block. Rows past the slice's last channel and pieces past
        // the reduction's end are zero.
        const int pj = (lane & 3) ^ lds_detail::swz(li);
        const uint8_t* wrow[NF];
        bool wrow_ok[NF];
        // (fragment f's row is 4 * f below fragment 0's: one 64-bit multiply, then uniform additions; rows past the
        // slice's last channel are never dereferenced)
        const uint8_t* const wrow0 = a.w + (int64_t)(oc0 + channel_of_frag_row<NF>(0, li)) * a.w_soc + pj * 16;
#pragma unroll
        for (int f = 0; f < NF; ++f) {
            wrow_ok[f] = channel_of_frag_row<NF>(f, li) < noc;
            wrow[f] = wrow0 + (int64_t)(4 * f) * a.w_soc;
        }
        // (an input zero point equal to the storage offset - u8 around 128 - makes every weight-sum term zero: no sums then)
        const bool need_sums = ASUM || a.da != 0;  // uniform
        int32_t wpart[NF];  // sum of the (signed) weights this lane staged, per channel fragment
#pragma unroll
        for (int f = 0; f < NF; ++f) wpart[f] = 0;
        constexpr int WB = NCE_WB;       // weight loads in flight per lane while staging
        constexpr int SB = WB / NF;  // steps per batch of loads
        uint4 v[SB][NF];
        // requests only (nothing here consumes a loaded value) ...
        auto request = [&](int s0) {
#pragma unroll
            for (int j = 0; j < SB; ++j) {
                const int st = s0 + j * nwaves;
                const bool in_k = st < S && 4 * st + pj < w.k16;
#pragma unroll
                for (int f = 0; f < NF; ++f) {
                    // (padding holds the XOR mask itself, so that the unconditional XOR below turns it into zero;
                    // nothing inside the branch may consume the loaded value, or the loads would serialise)
                    v[j][f] = make_uint4(a.w_xor, a.w_xor, a.w_xor, a.w_xor);
                    if (in_k && wrow_ok[f]) v[j][f] = *reinterpret_cast<const uint4*>(wrow[f] + (int64_t)st * 64);
                }
            }
        };
        // ... then the weight sums and LDS writes
        auto commit = [&](int s0) {
#pragma unroll
            for (int j = 0; j < SB; ++j) {
                const int st = s0 + j * nwaves;
                if (st < S) {  // uniform
#pragma unroll
                    for (int f = 0; f < NF; ++f) {
                        const uint4 sw = make_uint4(v[j][f].x ^ a.w_xor, v[j][f].y ^ a.w_xor, v[j][f].z ^ a.w_xor, v[j][f].w ^ a.w_xor);
                        if (need_sums) wpart[f] += bytesum(sw);
                        *reinterpret_cast<uint4*>(sWt + ((size_t)st * NF + f) * 1024 + lane * 16) = sw;
                    }
                }
            }
        };
        // The first weights go out before anything else; the pixel bookkeeping of the wave's first tile, its
        // first activation requests and the constants run while they are in flight.
        // (No branch around these activation requests - the wait for the weights would otherwise have to cover
        // them too; a wave without a tile requests the last pixel's data, which setup() clamps to.)
        WRES_MARK(0);
        request(wave);
        input_wait();
        setup();
        first_loads(false);
        WRES_MARK(1);
        if (consts_wave) do_consts();
        commit(wave);
        for (int s0 = wave + nwaves * SB; s0 < S; s0 += nwaves * SB) {
            request(s0);
            commit(s0);
        }
        // the four lanes of a row add up their pieces; the first of them publishes the wave's partial sum
#pragma unroll
        for (int f = 0; need_sums && f < NF; ++f) {
            int32_t p = wpart[f];
            p += __shfl_xor(p, 1);
            p += __shfl_xor(p, 2);
            if ((lane & 3) == 0) sWpart[wave][channel_of_frag_row<NF>(f, li)] = p;
        }
    }
    if constexpr (TBL) {
        for (int st = tid; st < S; st += (int)blockDim.x) sStep[st] = step_entry(st);
    } else if (MODE == WRES_GENERIC) {
        for (int u = tid; u < 4 * S; u += (int)blockDim.x) sStep[u] = unit_entry(u);
    }
    WRES_MARK(2);
    __syncthreads();  // weights and constants are in LDS; no workgroup synchronisation after this
    WRES_MARK(3);

    const int flags = sFlags;
    const PpeF64 pu = ppe_f64_setup(ppe_args, (flags & 2) != 0);
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
                // (through readfirstlane: otherwise the compiler replaces the sign-extended 32-bit value by the 64-bit q
                // it was cut from and multiplies 64 x 64 bits per output)
                ep.pmq = __builtin_amdgcn_readfirstlane((int32_t)q);
                ep.cpz = (half + zpf * ((int64_t)1 << ps) - zpf * pm) * ((int64_t)1 << (32 - ps));
            }
        }
    }
    // This wave's copy of the per-channel constants with the weight sums folded in (lane = channel). The
    // activation zero point enters as da * (sum of the channel's weights): |da| <= 255, |sum| < 2^23, and
    // the FP64 product and sum are exact (24 x 25 significant bits).
    if (lane < OCT) {
        int32_t ws = 0;
        // (an input zero point equal to the storage offset - u8 around 128 - makes every weight-sum term zero: no need to
        // collect the waves' partial sums then)
        if (ASUM || a.da != 0)
            for (int i = 0; i < nwaves; ++i) ws += sWpart[i][lane];
        // (with a weight zero-point offset dw the constant term S * 64 * da * dw joins; all below 2^30)
        const int32_t kdd = ASUM ? S * 64 * a.da * a.dw : 0;
        sCorr[wave][lane] = a.da * ws + kdd;
        double B = __builtin_fma((double)ws, sMd[lane], sBc[lane]);
        if (ASUM) B = __builtin_fma((double)kdd, sM[lane], B);
        if (pmode != PPE_MODE_INT) B += ep.zp_fold;  // floor(x + zp) = floor(x) + zp
        sBfull[wave][lane] = B;
        if (pmode == PPE_MODE_HI || pmode == PPE_MODE_HI_SLOPE) {
            const int32_t mult = table_mult(sW2[lane]), shift = table_shift(sW2[lane]);
            int32_t mq = 0;
            int64_t cq = 0;
            if (lane < noc) {  // (channels past the slice's end keep zeros; their results are not stored)
                const int64_t base = ((int64_t)sBias[lane] + sCorr[wave][lane]) * mult + ((int64_t)1 << (shift - 1))
                                   + ((int64_t)(pu.zp + (ep.flip ? 128 : 0)) << shift);
                mq = (int32_t)((uint32_t)mult << (32 - shift));
                cq = (int64_t)((uint64_t)base << (32 - shift));
            }
            sCorr[wave][lane] = mq;
            reinterpret_cast<int64_t*>(sBfull[wave])[lane] = cq;
        }
    }
    // (same wave writes and reads: program order is enough, the compiler waits on the LDS counter)

    // weights: lane (c16, q) reads piece q of row c16 of a block
    const int wfrag_off = c16 * 64 + (((lane >> 4) ^ lds_detail::swz(c16)) << 4);
    // ---- per-wave tile loop -----------------------------------------------------------------------
    WRES_MARK(4);
    while (t < t_end) {
        v4i acc[NF][BF];
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int x = 0; x < BF; ++x) acc[f][x] = v4i{0, 0, 0, 0};
        // Fused residual add: the other input's 16 channels of each of the lane's pixels are requested now and travel
        // while the reduction runs (unconditionally: a lane without a pixel or past the slice's last channel reads a
        // duplicate address inside the tensor).
        uint4 other[FZ ? BF : 1];
        if constexpr (FZ) {
            const int ch0 = min(16 * (lane >> 4), noc - 16);
#pragma unroll
            for (int x = 0; x < BF; ++x) other[x] = *reinterpret_cast<const uint4*>(w.fz.other + ((dst[x] + ch0) - a.out));
        }
        // Steady state: every step consumes one ring slot and refills it for step + D, with no branch
        // around the load, so that the wait before a step covers exactly the loads older than its own.
        v4i asum[BF];
#pragma unroll
        for (int x = 0; x < BF; ++x) asum[x] = v4i{0, 0, 0, 0};
        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
        const uint8_t* ap = sWt + wfrag_off;
        v4i fa[NF];
#pragma unroll
        for (int f = 0; f < NF; ++f) fa[f] = *reinterpret_cast<const v4i*>(ap + f * 1024);
        auto mma = [&](const v4i (&braw)[BF], bool more_a) {
            v4i b[BF];
#pragma unroll
            for (int x = 0; x < BF; ++x) b[x] = braw[x] ^ axor;
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int x = 0; x < BF; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[f], b[x], acc[f][x], 0, 0, 0);
            if constexpr (ASUM) {
#pragma unroll
                for (int x = 0; x < BF; ++x) asum[x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, b[x], asum[x], 0, 0, 0);
            }
            ap += NF * 1024;
            if (more_a) {
#pragma unroll
                for (int f = 0; f < NF; ++f) fa[f] = *reinterpret_cast<const v4i*>(ap + f * 1024);
            }
        };
        if constexpr (TRL) {
            // The permute of step s + 1 is issued before the matrix instructions of step s, so its latency
            // hides behind them; a ring slot is free for its next load once its permute has been issued.
            auto to_operand = [&](const v4i (&raw)[BF], v4i (&o)[BF]) {
#pragma unroll
                for (int x = 0; x < BF; ++x)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[x][r] = __builtin_amdgcn_ds_bpermute(to_mfma, raw[x][r]);
            };
            v4i cur[BF], nxt[BF];
            to_operand(fb[0], cur);
            for (int g = D; g < S; g += D) {
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    to_operand(fb[(j + 1) % D], nxt);
                    load_b(fb[j]);
                    mma(cur, true);
#pragma unroll
                    for (int x = 0; x < BF; ++x) cur[x] = nxt[x];
                }
            }
#pragma unroll
            for (int j = 0; j < D; ++j) {
                if (j + 1 < D) to_operand(fb[j + 1], nxt);
                mma(cur, j + 1 < D);
#pragma unroll
                for (int x = 0; x < BF; ++x) cur[x] = nxt[x];
            }
        } else {
            if constexpr (D > 1) {  // (depth 1 is launched for single-step reductions only: the zeroed
                                    // accumulators then fold into the one matrix instruction's addend)
                for (int g = D; g < S; g += D) {
#pragma unroll
                    for (int j = 0; j < D; ++j) {
                        mma(fb[j], true);
                        load_b(fb[j]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < D; ++j) mma(fb[j], j + 1 < D);
        }
        int32_t dws[BF];  // every row of asum holds the pixel's sum: register 0 of this lane is its column's
#pragma unroll
        for (int x = 0; x < BF; ++x) dws[x] = ASUM ? a.dw * asum[x][0] : 0;
        WRES_MARK(5);  // (of the wave's last tile)
        if (pmode == PPE_MODE_HI) wres_epilogue<NF, BF, PPE_MODE_HI, FZ>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep, &w.fz, other);
        else if (pmode == PPE_MODE_HI_SLOPE) wres_epilogue<NF, BF, PPE_MODE_HI_SLOPE, FZ>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep, &w.fz, other);
        else if (pmode == PPE_MODE_FOLDED) wres_epilogue<NF, BF, PPE_MODE_FOLDED, FZ>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep, &w.fz, other);
        else if (pmode == PPE_MODE_SLOPE) wres_epilogue<NF, BF, PPE_MODE_SLOPE, FZ>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep, &w.fz, other);
        else wres_epilogue<NF, BF, PPE_MODE_INT, FZ>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep, &w.fz, other);
        t += nwaves;
        if (t < t_end) {
            setup();
            first_loads(true);
        }
    }
    WRES_MARK(6);
}

template <int NF, int BF, int MODE, int D, int LM>
__global__ __launch_bounds__(512) void conv_wres_kernel(WresArgs w) {
    prefetch_kernel_arguments<sizeof(WresArgs)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t sWt[];  // [step][fragment][lane] x 16 bytes
    __shared__ WresSmemOf<NF, MODE> sm;
    const uint32_t group = xcd_tile(blockIdx.x, w.ngroups);
    if (group >= w.ngroups) return;  // uniform for the whole workgroup
    conv_wres_body<NF, BF, MODE, D, LM>(w, group, blockIdx.y, sWt, sm, NoInputWait{});
}

constexpr int wres_tag(int nf, int bf, int mode, int d, int lm) {
    return nf * 10000 + bf * 1000 + mode * 100 + d * 10 + lm;
}

constexpr size_t kWresLdsCap = 144 * 1024;  // dynamic LDS one workgroup may take (160 KiB per CU less tables)

template <int NF, int BF, int MODE, int D, int LM>
hipError_t launch_one(WresArgs& w, int nwaves, int tiles_per_wave, hipStream_t stream) {
    constexpr int OCT = 16 * NF;
    constexpr int BP = 16 * BF;
    const ConvArgs& a = w.a;
    w.ntiles = (uint32_t)(((int64_t)a.M + BP - 1) / BP);
    if (w.tpg == 0) w.tpg = nwaves * tiles_per_wave;  // (the caller may have chosen a tile count per workgroup that is no multiple)
    w.ngroups = (w.ntiles + w.tpg - 1) / w.tpg;
    const unsigned gy = (unsigned)((a.bc + OCT - 1) / OCT);
    w.nsteps = (w.nsteps + D - 1) / D * D;
    const size_t lds = (size_t)w.nsteps * NF * 1024;
    if (lds > kWresLdsCap || w.nsteps > kMaxSteps) return hipErrorNotSupported;
    if (MODE == WRES_GENERIC && lds > kWresLdsCap - 4096) return hipErrorNotSupported;  // its step table is 4 KiB larger
    auto kernel = &conv_wres_kernel<NF, BF, MODE, D, LM>;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    // (the tag names the instantiation for the persistent form, which runs eight waves)
    return emit(kernel, dim3(xcd_grid(w.ngroups), gy), dim3(64 * nwaves), lds, stream, w, nwaves == 8 ? wres_tag(NF, BF, MODE, D, LM) : 0);
}

template <int NF, int BF, int D>
hipError_t launch_depth(WresArgs& w, int mode, int nwaves, int tpw, hipStream_t stream) {
    // Transposed loads: measured to pay for every kernel larger than 1x1 and for long 1x1 reductions, once
    // pixels are more than 64 bytes apart (the per-lane mode serves channel counts below that).
    const bool trl = D >= 2 && mode != WRES_GENERIC && w.a.in_sw > 64 && (w.ntaps > 1 || w.nsteps >= 32);
    if (w.fused) {
        // The fused residual add exists for the 64-channel kernels with plain loads and every tap inside the image
        // (the 1x1 convolutions that close a residual block).
        if constexpr (NF == 4) {
            if (mode == WRES_FAST && !trl && w.a.dw == 0 && w.a.out_sc == 1) return launch_one<NF, BF, WRES_FAST, D, LM_PLAIN_FZ>(w, nwaves, tpw, stream);
        }
        return hipErrorNotSupported;
    }
    if constexpr (D == 1 || D == 2 || D == 4) {
        if (w.a.dw != 0) {  // activation sums for the weight zero-point term
            if constexpr (D >= 2) {
                if (trl && mode == WRES_FAST) return launch_one<NF, BF, WRES_FAST, D, LM_TRL_ASUM>(w, nwaves, tpw, stream);
                if (trl && mode == WRES_FAST_MASK) return launch_one<NF, BF, WRES_FAST_MASK, D, LM_TRL_ASUM>(w, nwaves, tpw, stream);
            }
            if (mode == WRES_FAST) return launch_one<NF, BF, WRES_FAST, D, LM_PLAIN_ASUM>(w, nwaves, tpw, stream);
            if (mode == WRES_FAST_MASK) return launch_one<NF, BF, WRES_FAST_MASK, D, LM_PLAIN_ASUM>(w, nwaves, tpw, stream);
            return launch_one<NF, BF, WRES_GENERIC, D, LM_PLAIN_ASUM>(w, nwaves, tpw, stream);
        }
    }
    if (w.a.dw != 0) return hipErrorNotSupported;  // (launch_mode sends those tasks to depth 1, 2 or 4)
    if constexpr (D >= 2) {
        if (trl && mode == WRES_FAST) return launch_one<NF, BF, WRES_FAST, D, LM_TRL>(w, nwaves, tpw, stream);
        if (trl && mode == WRES_FAST_MASK) return launch_one<NF, BF, WRES_FAST_MASK, D, LM_TRL>(w, nwaves, tpw, stream);
        // step table: every step changes tap
        const bool tbl = w.ntaps > 1 && w.nc64 == 1;
        if (tbl && mode == WRES_FAST) return launch_one<NF, BF, WRES_FAST, D, LM_TBL>(w, nwaves, tpw, stream);
        if (tbl && mode == WRES_FAST_MASK) return launch_one<NF, BF, WRES_FAST_MASK, D, LM_TBL>(w, nwaves, tpw, stream);
    }
    if (mode == WRES_FAST) return launch_one<NF, BF, WRES_FAST, D, LM_PLAIN>(w, nwaves, tpw, stream);
    if (mode == WRES_FAST_MASK) return launch_one<NF, BF, WRES_FAST_MASK, D, LM_PLAIN>(w, nwaves, tpw, stream);
    return launch_one<NF, BF, WRES_GENERIC, D, LM_PLAIN>(w, nwaves, tpw, stream);
}

template <int NF, int BF>
hipError_t launch_mode(WresArgs& w, int mode, int nwaves, int tpw, hipStream_t stream) {
    if (w.a.dw != 0) {
        // Depth 4 or 2 only (1 for a single-step reduction). A padding step must read the fill line (its
        // activations enter the pixel sums), which the mask mode guarantees: its tap bit is clear.
        if (w.nsteps == 1) return launch_depth<NF, BF, 1>(w, mode, nwaves, tpw, stream);
        constexpr bool d4 = BF < 4;
        const bool pad = !(d4 && w.nsteps % 4 == 0) && w.nsteps % 2 != 0;
        if (pad && mode == WRES_FAST) {
            if (w.ntaps > 31) return hipErrorNotSupported;
            mode = WRES_FAST_MASK;
        }
        if constexpr (d4) {
            if (w.nsteps % 4 == 0) return launch_depth<NF, BF, 4>(w, mode, nwaves, tpw, stream);
        }
        return launch_depth<NF, BF, 2>(w, mode, nwaves, tpw, stream);
    }
    // Load depth: the deepest of 4, 3, 2 steps that needs no padding step and whose ring fits the registers;
    // a single-step reduction (1x1 kernel over 64 channels) runs without ring or padding.
    if (w.nsteps == 1) return launch_depth<NF, BF, 1>(w, mode, nwaves, tpw, stream);
    if constexpr (BF < 4) {
        if (w.nsteps % 4 == 0) return launch_depth<NF, BF, 4>(w, mode, nwaves, tpw, stream);
        if (w.nsteps % 3 == 0) return launch_depth<NF, BF, 3>(w, mode, nwaves, tpw, stream);
    } else {
        // 64-pixel tiles: depth 3 only where depth 2 would need a padding step (9 steps: 3x3 over 64 channels)
        if (w.nsteps % 2 != 0 && w.nsteps % 3 == 0) return launch_depth<NF, BF, 3>(w, mode, nwaves, tpw, stream);
    }
    return launch_depth<NF, BF, 2>(w, mode, nwaves, tpw, stream);
}

#if WRES_PART == 0
// ---- reductions longer than LDS: the same kernel shape with the weights staged chunk by chunk ------------
// For slices whose reduction does not fit LDS (3x3 over 1024 channels, 5x5 over 256, 1x1 over 8192 ...) the
// workgroup stages CS steps of its weights, synchronises, lets every wave run those steps on its (single) tile,
// synchronises again and stages the next chunk; accumulators and the activation ring live across chunks.
// Kept simple: 64-byte-aligned input channels, one tile per wave, load depth 4, permuted activation loads, scalar
// tap counters, row / column validity bits (any kernel up to 31 x 31). ASUM as in conv_wres_kernel.
template <int NF, int BF, bool ASUM>
__global__ __launch_bounds__(512) void conv_wres_chunked_kernel(WresArgs w) {
    prefetch_kernel_arguments<sizeof(WresArgs)>();
    constexpr int OCT = 16 * NF;
    constexpr int BP = 16 * BF;
    constexpr int D = 4;
    constexpr int WB = 4;
    const ConvArgs& a = w.a;

    extern __shared__ __attribute__((aligned(16))) uint8_t sWt[];  // one chunk: [step][fragment][lane] x 16 bytes
    __shared__ int32_t sW2[OCT], sBias[OCT];
    __shared__ double sM[OCT], sBc[OCT], sMd[OCT];
    __shared__ int32_t sWpart[8][OCT];
    __shared__ int32_t sCorr[8][OCT];
    __shared__ double sBfull[8][OCT];
    __shared__ int32_t sFlags;
    const EpiSmem es = {sM, sBc, sW2, sBias, nullptr, nullptr};

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = blockDim.x >> 6;
    const int c16 = lane & 15;
    const int pl = lane >> 2, kc = lane & 3;          // pixel and 16-byte piece this lane loads
    const int to_mfma = 4 * (4 * c16 + (lane >> 4));  // ds_bpermute source: lane 4p + k feeds lane 16k + p

    const int32_t oc0 = a.z0 + blockIdx.y * OCT;
    const int32_t noc = min(OCT, a.z0 + a.bc - oc0);
    const uint32_t group = xcd_tile(blockIdx.x, w.ngroups);
    if (group >= w.ngroups) return;  // uniform for the whole workgroup

    const int axor = (int)a.a_xor;
    const uint8_t* const fillp = &g_fill.b[(a.fill ^ a.a_xor) & 0xFFu][kc * 16];
    const int S = w.nsteps;   // padded to a multiple of D
    const int CS = w.cs;      // steps per chunk, a multiple of D
    const uint32_t t = group * (uint32_t)w.tpg + wave;  // this wave's tile (one per wave)
    const bool has_tile = t < w.ntiles;

    // ---- the tile: pixel addresses and validity bits (a wave without a tile works on the last pixel, stores nothing)
    const uint8_t* pbase[BF];
    uint8_t* dst[BF];
    bool valid[BF];
    uint32_t rows[BF], cols[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) {
        const uint32_t p = t * BP + 16 * x + pl;
        const bool in_range = p < (uint32_t)a.M;
        const int32_t pc = in_range ? (int32_t)p : a.M - 1;
        const int32_t rr = fdiv(pc, a.div_bw);
        const int32_t bx = pc - rr * a.bw;
        const int32_t n = fdiv(rr, a.div_bh);
        const int32_t by = rr - n * a.bh;
        const int32_t iy0 = (a.y0 + by) * a.SY - a.PT;
        const int32_t ix0 = (a.x0 + bx) * a.SX - a.PL;
        pbase[x] = a.in + (int64_t)n * a.in_sn + (int64_t)iy0 * a.in_sh + (int64_t)ix0 * a.in_sw + kc * 16;
        uint8_t* d = a.out + (int64_t)n * a.out_sn + (int64_t)(a.y0 + by) * a.out_sh + (int64_t)(a.x0 + bx) * a.out_sw + oc0 * a.out_sc;
        // results come out in matrix layout: take the address of pixel c16 from a lane that computed it
        const uint64_t dl = reinterpret_cast<uint64_t>(d);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(16 * c16, (int)(uint32_t)dl);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(16 * c16, (int)(uint32_t)(dl >> 32));
        dst[x] = reinterpret_cast<uint8_t*>(((uint64_t)hi << 32) | lo);
        valid[x] = has_tile && t * BP + 16 * x + c16 < (uint32_t)a.M;
        rows[x] = bit_range(max(0, -iy0), min(a.KY, a.H - iy0));  // bit 31 stays clear (KY, KX <= 31): padding steps
        cols[x] = bit_range(max(0, -ix0), min(a.KX, a.W - ix0));
    }
    // scalar walk over (kernel row, kernel column, 64-byte channel chunk); additions only
    int32_t it_ky = 0, it_kx = 0, it_c64 = 0;
    int64_t it_off = 0, tap_off = 0;
    v4i fb[D][BF];
    auto load_b = [&](v4i (&d)[BF]) {
#pragma unroll
        for (int x = 0; x < BF; ++x) {
            const uint8_t* src = pbase[x] + it_off;
            src = ((rows[x] >> it_ky) & (cols[x] >> it_kx) & 1u) ? src : fillp;
            d[x] = *reinterpret_cast<const v4i*>(src);
        }
        it_off += 64;
        if (++it_c64 == w.nc64) {
            it_c64 = 0;
            tap_off += a.in_sw;
            if (++it_kx == a.KX) {
                it_kx = 0;
                tap_off += w.row_adv;
                if (++it_ky >= a.KY) {  // padding steps: a readable address, a clear validity bit
                    it_ky = 31;
                    tap_off = 0;
                }
            }
            it_off = tap_off;
        }
    };

    // ---- weight staging (see conv_wres_kernel) ---------------------------------------------------------------
    const int li = lane >> 2, lk = (lane & 3) ^ lds_detail::swz(li);  // row and piece this lane stages (blocks stay row-major)
    const int64_t acc_bound = min((int64_t)a.ktot * 65025, (int64_t)2147483648LL);
    const bool consts_wave = wave == nwaves - 1;
    int32_t tw2 = 0, tbias = 0;
    if (consts_wave && lane < noc) {
        const int32_t* trow = a.table + (int64_t)(oc0 + lane) * a.table_stride;
        tw2 = trow[2];
        tbias = trow[3];
    }
    const uint8_t* wrow[NF];
    bool wrow_ok[NF];
    const uint8_t* const wrow0 = a.w + (int64_t)(oc0 + channel_of_frag_row<NF>(0, li)) * a.w_soc + lk * 16;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        wrow_ok[f] = channel_of_frag_row<NF>(f, li) < noc;
        wrow[f] = wrow0 + (int64_t)(4 * f) * a.w_soc;
    }
    int32_t wpart[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) wpart[f] = 0;
    constexpr int SB = WB / NF;
    uint4 v[SB][NF];
    auto request = [&](int s0, int send) {
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            const int st = s0 + j * nwaves;
            const bool in_k = st < send && 4 * st + lk < w.k16;
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                v[j][f] = make_uint4(a.w_xor, a.w_xor, a.w_xor, a.w_xor);  // (becomes zero under the XOR below)
                if (in_k && wrow_ok[f]) v[j][f] = *reinterpret_cast<const uint4*>(wrow[f] + (int64_t)st * 64);
            }
        }
    };
    auto commit = [&](int s0, int sbase, int send) {
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            const int st = s0 + j * nwaves;
            if (st < send) {  // uniform
#pragma unroll
                for (int f = 0; f < NF; ++f) {
                    const uint4 sw = make_uint4(v[j][f].x ^ a.w_xor, v[j][f].y ^ a.w_xor, v[j][f].z ^ a.w_xor, v[j][f].w ^ a.w_xor);
                    if (ASUM || a.da != 0) wpart[f] += bytesum(sw);  // (uniform: no sums when the input zero-point term is zero)
                    *reinterpret_cast<uint4*>(sWt + ((size_t)(st - sbase) * NF + f) * 1024 + lane * 16) = sw;
                }
            }
        }
    };
    auto stage_chunk = [&](int sbase, int send) {
        for (int s0 = sbase + wave; s0 < send; s0 += nwaves * SB) {
            request(s0, send);
            commit(s0, sbase, send);
        }
    };

    // first chunk: the activation requests of the first D steps go out while its first weights are in flight
    const int send0 = min(CS, S);
    request(wave, send0);
#pragma unroll
    for (int j = 0; j < D; ++j) load_b(fb[j]);
    if (consts_wave) {
        const int32_t mult = table_mult(tw2), shift = table_shift(tw2);
        const bool bad = lane < OCT && shift > kMaxF64Shift;
        const bool sat = lane < OCT && ppe_may_saturate(acc_bound, tbias, mult, shift);
        const int wf = (__any(bad) ? 1 : 0) | (__any(sat) ? 2 : 0);
        if (lane == 0) sFlags = wf;
        if (lane < OCT) {
            const double M = ppe_scale_M(mult, shift);
            sW2[lane] = tw2;
            sBias[lane] = tbias;
            sM[lane] = M;
            sMd[lane] = M * (double)a.da;
            sBc[lane] = ppe_scale_B(tbias, M, shift, a.ppe.round_mode);
        }
    }
    commit(wave, 0, send0);
    for (int s0 = wave + nwaves * SB; s0 < send0; s0 += nwaves * SB) {
        request(s0, send0);
        commit(s0, 0, send0);
    }

    // ---- chunks ------------------------------------------------------------------------------------------------
    v4i acc[NF][BF];
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int x = 0; x < BF; ++x) acc[f][x] = v4i{0, 0, 0, 0};
    auto to_operand = [&](const v4i (&raw)[BF], v4i (&o)[BF]) {
#pragma unroll
        for (int x = 0; x < BF; ++x)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[x][r] = __builtin_amdgcn_ds_bpermute(to_mfma, raw[x][r]);
    };
    v4i cur[BF], nxt[BF];
    to_operand(fb[0], cur);
    v4i asum[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) asum[x] = v4i{0, 0, 0, 0};
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    for (int sbase = 0; sbase < S; sbase += CS) {
        const int send = min(sbase + CS, S);
        if (sbase > 0) stage_chunk(sbase, send);
        if (send == S) {  // every weight has passed through: publish the wave's partial sums
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                int32_t p = wpart[f];
                p += __shfl_xor(p, 1);
                p += __shfl_xor(p, 2);
                if (lk == 0) sWpart[wave][channel_of_frag_row<NF>(f, li)] = p;
            }
        }
        __syncthreads();  // the chunk is in LDS
        const uint8_t* ap = sWt + (lane & 15) * 64 + (((lane >> 4) ^ lds_detail::swz(lane & 15)) << 4);  // piece lane / 16 of row lane % 16
        v4i fa[NF];
#pragma unroll
        for (int f = 0; f < NF; ++f) fa[f] = *reinterpret_cast<const v4i*>(ap + f * 1024);
        auto mma = [&](bool more_a) {
            v4i b[BF];
#pragma unroll
            for (int x = 0; x < BF; ++x) b[x] = cur[x] ^ axor;
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int x = 0; x < BF; ++x) acc[f][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[f], b[x], acc[f][x], 0, 0, 0);
            if constexpr (ASUM) {
#pragma unroll
                for (int x = 0; x < BF; ++x) asum[x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, b[x], asum[x], 0, 0, 0);
            }
            ap += NF * 1024;
            if (more_a) {
#pragma unroll
                for (int f = 0; f < NF; ++f) fa[f] = *reinterpret_cast<const v4i*>(ap + f * 1024);
            }
        };
        for (int g = sbase; g < send; g += D) {
            const bool last_in_chunk = g + D >= send;
            if (g + D < S) {  // uniform: steps remain after this group, its ring slots are refilled
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    to_operand(fb[(j + 1) % D], nxt);
                    load_b(fb[j]);
                    mma(!(last_in_chunk && j == D - 1));
#pragma unroll
                    for (int x = 0; x < BF; ++x) cur[x] = nxt[x];
                }
            } else {
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    if (j + 1 < D) to_operand(fb[j + 1], nxt);
                    mma(j + 1 < D);
#pragma unroll
                    for (int x = 0; x < BF; ++x) cur[x] = nxt[x];
                }
            }
        }
        if (send < S) __syncthreads();  // every wave is done with the chunk before it is overwritten
    }

    const int flags = sFlags;
    const PpeF64 pu = ppe_f64_setup(a.ppe, (flags & 2) != 0);
    const int pmode = ppe_mode_of(pu, (flags & 1) != 0);
    const EpiPack ep = epi_pack_setup(pu);
    if (lane < OCT) {
        int32_t ws = 0;
        // (an input zero point equal to the storage offset - u8 around 128 - makes every weight-sum term zero: no need to
        // collect the waves' partial sums then)
        if (ASUM || a.da != 0)
            for (int i = 0; i < nwaves; ++i) ws += sWpart[i][lane];
        // (the host rejects reductions for which S * 64 * da * dw or dw * a pixel's sum could leave int32)
        const int32_t kdd = ASUM ? S * 64 * a.da * a.dw : 0;
        sCorr[wave][lane] = a.da * ws + kdd;
        double B = __builtin_fma((double)ws, sMd[lane], sBc[lane]);
        if (ASUM) B = __builtin_fma((double)kdd, sM[lane], B);
        if (pmode != PPE_MODE_INT) B += ep.zp_fold;
        sBfull[wave][lane] = B;
    }
    int32_t dws[BF];
#pragma unroll
    for (int x = 0; x < BF; ++x) dws[x] = ASUM ? a.dw * asum[x][0] : 0;
    if (pmode == PPE_MODE_FOLDED) wres_epilogue<NF, BF, PPE_MODE_FOLDED>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep);
    else if (pmode == PPE_MODE_SLOPE) wres_epilogue<NF, BF, PPE_MODE_SLOPE>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep);
    else wres_epilogue<NF, BF, PPE_MODE_INT>(a, es, sBfull[wave], sCorr[wave], acc, dws, lane >> 4, noc, dst, valid, pu, ep);
}

template <int NF, int BF, bool ASUM>
hipError_t launch_chunked(WresArgs& w, int nwaves, hipStream_t stream) {
    constexpr int OCT = 16 * NF;
    constexpr int BP = 16 * BF;
    const ConvArgs& a = w.a;
    w.ntiles = (uint32_t)(((int64_t)a.M + BP - 1) / BP);
    w.tpg = nwaves;  // one tile per wave
    w.ngroups = (w.ntiles + w.tpg - 1) / w.tpg;
    const unsigned gy = (unsigned)((a.bc + OCT - 1) / OCT);
    w.nsteps = (w.nsteps + 3) / 4 * 4;
    w.cs = (int32_t)(kWresLdsCap / ((size_t)NF * 1024)) / 4 * 4;
    const size_t lds = (size_t)std::min(w.cs, w.nsteps) * NF * 1024;
    auto kernel = &conv_wres_chunked_kernel<NF, BF, ASUM>;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    return emit(kernel, dim3(xcd_grid(w.ngroups), gy), dim3(64 * nwaves), lds, stream, w);
}

// Long reductions: 32 channels x 72 steps per chunk; the pixel tile as large as still gives ~1500 wave tiles.
hipError_t launch_conv_wres_chunked(WresArgs& w, hipStream_t stream) {
    const ConvArgs& a = w.a;
    if (a.IC % 64 != 0 || a.KY > 31 || a.KX > 31) return hipErrorNotSupported;
    // (weight zero-point offset: keep S * 64 * da * dw and dw * pixel sums inside int32 for the integer PPE path)
    if (a.dw != 0 && (int64_t)(w.nsteps + 3) * 64 * 255 * 255 > 0x7fffffffLL) return hipErrorNotSupported;
    const int64_t slices = (a.bc + 31) / 32;
    int bf = (((int64_t)a.M + 31) / 32) * slices >= 1500 ? 2 : 1;
    int nw = 8;
    if (options().wres_forced) {  // "nf,bf,nwaves,tiles_per_wave": bf (1, 2) and nwaves apply
        const int fbf = options().wres[1], fnw = options().wres[2];
        if (fbf == 1 || fbf == 2) bf = fbf;
        if (fnw >= 1 && fnw <= 8) nw = fnw;
    }
    if (a.dw != 0) return bf == 2 ? launch_chunked<2, 2, true>(w, nw, stream) : launch_chunked<2, 1, true>(w, nw, stream);
    return bf == 2 ? launch_chunked<2, 2, false>(w, nw, stream) : launch_chunked<2, 1, false>(w, nw, stream);
}

#endif  // WRES_PART == 0

template <int NF>
hipError_t launch_bf(WresArgs& w, int bf, int mode, int nwaves, int tpw, hipStream_t stream) {
    if (bf == 4) return launch_mode<NF, 4>(w, mode, nwaves, tpw, stream);
    if (bf == 2) return launch_mode<NF, 2>(w, mode, nwaves, tpw, stream);
    return launch_mode<NF, 1>(w, mode, nwaves, tpw, stream);
}

}  // namespace

#if WRES_PART == 1
hipError_t launch_wres_nf4_bf4(WresArgs& w, int mode, int nwaves, int tpw, hipStream_t stream);
hipError_t launch_wres_nf4(WresArgs& w, int bf, int mode, int nwaves, int tpw, hipStream_t stream) {
    if (bf == 4) return launch_wres_nf4_bf4(w, mode, nwaves, tpw, stream);
    if (bf == 2) return launch_mode<4, 2>(w, mode, nwaves, tpw, stream);
    return launch_mode<4, 1>(w, mode, nwaves, tpw, stream);
}
#elif WRES_PART == 2
hipError_t launch_wres_nf4_bf4(WresArgs& w, int mode, int nwaves, int tpw, hipStream_t stream) {
    return launch_mode<4, 4>(w, mode, nwaves, tpw, stream);
}
#elif WRES_PART == 0
#ifdef WRES_TRACE
uint64_t* g_wres_trace = nullptr;
uint32_t g_wres_trace_seq = 0;
extern "C" void nceProbeSetWresTrace(uint64_t* device_buffer) {
    g_wres_trace = device_buffer;
    g_wres_trace_seq = 0;
}
#endif
hipError_t launch_conv_wres(const ConvArgs& a, hipStream_t stream, bool allow_chunked, const FuseAdd* fuse) {
    if (a.KY > 32 || a.KX > 32) return hipErrorNotSupported;
    // (pixel indices of tiles past the end - waves without a tile still form addresses - must stay below 2^31)
    if (a.M > 0x7fffffff - 64 * 1024) return hipErrorNotSupported;
    WresArgs w;
#ifdef WRES_TRACE
    w.trace = g_wres_trace != nullptr ? g_wres_trace + (size_t)(g_wres_trace_seq++ % 64) * 256 * 8 * 8 : nullptr;
#endif
    w.a = a;
    w.fused = fuse != nullptr;
    if (fuse) w.fz = *fuse;
    else memset(&w.fz, 0, sizeof(w.fz));
    w.k16 = a.KG;
    w.nsteps = (a.KG + 3) / 4;
    w.nc64 = a.IC / 64;
    w.ntaps = a.KY * a.KX;
    w.div_icg = make_fastdiv((uint32_t)a.ICG);
    w.div_kx = make_fastdiv((uint32_t)a.KX);
    w.div_nc64 = make_fastdiv((uint32_t)std::max(1, w.nc64));
    w.row_adv = a.in_sh - (int64_t)a.KX * a.in_sw;
    for (const int64_t st : {a.in_sn, a.in_sh, a.in_sw, a.out_sn, a.out_sh, a.out_sw})
        if (st < 0 || st > 0x7fffffffLL) return hipErrorNotSupported;
    w.in_sn32 = (int32_t)a.in_sn;
    w.in_sh32 = (int32_t)a.in_sh;
    w.in_sw32 = (int32_t)a.in_sw;
    w.out_sn32 = (int32_t)a.out_sn;
    w.out_sh32 = (int32_t)a.out_sh;
    w.out_sw32 = (int32_t)a.out_sw;
    const size_t wl4 = (size_t)((w.nsteps + 1) / 2 * 2) * 4 * 1024, wl2 = wl4 / 2;  // with the padding step
    if (wl2 > kWresLdsCap) return allow_chunked && !w.fused ? launch_conv_wres_chunked(w, stream) : hipErrorNotSupported;

    // every tap of every output pixel of the box inside the image?
    const int64_t iy_lo = (int64_t)a.y0 * a.SY - a.PT, iy_hi = (int64_t)(a.y0 + a.bh - 1) * a.SY - a.PT + a.KY - 1;
    const int64_t ix_lo = (int64_t)a.x0 * a.SX - a.PL, ix_hi = (int64_t)(a.x0 + a.bw - 1) * a.SX - a.PL + a.KX - 1;
    const bool inside = iy_lo >= 0 && iy_hi < a.H && ix_lo >= 0 && ix_hi < a.W;
    const int mode = (a.IC % 64 != 0) ? WRES_GENERIC : (inside ? WRES_FAST : WRES_FAST_MASK);
    w.linear = a.KY == 1 && a.KX == 1 && a.SY == 1 && a.SX == 1 && a.PT == 0 && a.PL == 0 && a.x0 == 0 && a.y0 == 0 &&
               a.bw == a.W && a.bh == a.H && a.in_sh == (int64_t)a.W * a.in_sw && a.in_sn == (int64_t)a.H * a.in_sh &&
               a.out_sh == (int64_t)a.bw * a.out_sw && a.out_sn == (int64_t)a.bh * a.out_sh;
    // one bit per tap, bit 31 stays clear; larger kernels take the chunked kernel's row / column bits
    if (mode == WRES_FAST_MASK && a.KY * a.KX > 31) return allow_chunked && !w.fused ? launch_conv_wres_chunked(w, stream) : hipErrorNotSupported;

    // Shape of the work: nf channel fragments per slice, bf pixel fragments per wave tile. Measured on
    // MI355X over the ResNet-50 layer shapes, the best shape is always the LARGEST tile that still
    // yields about 1500 wave tiles (six waves per CU, one round of workgroups); beyond that, waves take
    // several tiles each rather than the grid growing.
    auto wave_tiles = [&](int nf, int bf) {
        return (((int64_t)a.M + 16 * bf - 1) / (16 * bf)) * ((a.bc + 16 * nf - 1) / (16 * nf));
    };
    const bool nf4_ok = wl4 <= kWresLdsCap && a.bc > 32;
    // (1x1 kernels over more than 64 input channels: measured faster with smaller pixel tiles, about 24 per CU)
    // (per-XCD form: an eighth of the work on an eighth of the CUs - the same choices as for the whole task)
    const int cus = tls_launch.per_xcd ? 32 : 256;
    const int64_t want = ((w.ntaps == 1 && w.nsteps > 1) ? 6000 : 1500) * cus / 256;
    // (per-XCD form: tiles of at most 32 pixels - the persistent kernel carries no 64-pixel instantiation, whose registers
    // every layer's path would pay for)
    int nf = nf4_ok ? 4 : 2, bf = tls_launch.per_xcd ? 2 : 4;
    while (bf > 1 && wave_tiles(nf, bf) < want) bf >>= 1;
    if (nf == 4 && wave_tiles(nf, bf) < 1500 * cus / 256) nf = 2;
    const int nwaves = 8;
    int tpw = 1;
    // Tiles per workgroup: one workgroup per CU where the tiles reach that far (the waves of a workgroup then
    // take unequal numbers of tiles, which costs less than leaving CUs idle or queueing a second round).
    const auto pick_tpg = [&](int nf_, int bf_, int nw_) {
        const int64_t ntiles = ((int64_t)a.M + 16 * bf_ - 1) / (16 * bf_);
        const int64_t slices = (a.bc + 16 * nf_ - 1) / (16 * nf_);
        const int64_t groups = std::max<int64_t>(1, cus / slices);
        return (uint32_t)std::max<int64_t>(nw_, (ntiles + groups - 1) / groups);
    };

    int nw = nwaves;
    bool forced_tpw = false;
    if (options().wres_forced) {  // tuning and test knob: "nf,bf,nwaves,tiles_per_wave"
        const int fnf = options().wres[0], fbf = options().wres[1], fnw = options().wres[2], ftpw = options().wres[3];
        if ((fnf == 2 || (fnf == 4 && wl4 <= kWresLdsCap))) nf = fnf;
        if (fbf == 1 || fbf == 2 || fbf == 4) bf = fbf;
        if (fnw >= 1 && fnw <= 8) nw = fnw;
        if (ftpw >= 1) tpw = ftpw, forced_tpw = true;  // (0: keep the automatic choice below)
    }
    if (w.fused && nf4_ok) nf = 4;  // (the fused add exists for the 64-channel kernels)
    w.tpg = forced_tpw ? 0 : pick_tpg(nf, bf, nw);
    if (nf == 4) return launch_wres_nf4(w, bf, mode, nw, tpw, stream);
    return launch_bf<2>(w, bf, mode, nw, tpw, stream);
}
#endif  // WRES_PART

#if WRES_PART == 3
// ---- persistent segments (nce_conv_pk.h) ---------------------------------------------------------------------------------
namespace {

// The instantiations a segment may use: NF, BF, MODE, D, LM (those of the ResNet-50 bottleneck layers at 4 images per XCD).
#define WRES_PK_VARIANTS(X)                                                                                           \
    X(0, 4, 1, WRES_FAST, 4, LM_PLAIN) X(1, 4, 1, WRES_FAST, 4, LM_PLAIN_FZ) X(2, 4, 1, WRES_FAST_MASK, 4, LM_TRL)     \
    X(4, 2, 1, WRES_FAST_MASK, 4, LM_TRL) X(5, 4, 2, WRES_FAST_MASK, 3, LM_TRL)  \
    X(6, 4, 2, WRES_FAST, 2, LM_PLAIN_FZ) X(8, 2, 1, WRES_FAST, 4, LM_TRL)      \
    X(10, 4, 2, WRES_FAST, 4, LM_PLAIN_FZ) X(11, 4, 2, WRES_FAST, 4, LM_PLAIN)     \
    X(12, 4, 2, WRES_FAST, 2, LM_PLAIN) X(13, 4, 2, WRES_FAST, 1, LM_PLAIN) X(14, 4, 2, WRES_FAST, 1, LM_PLAIN_FZ)          \
    X(15, 4, 2, WRES_FAST_MASK, 3, LM_TBL)

// Device table: [xcd][layer], the launch arguments of that XCD's share (pointers already advanced to its images).
struct PkLayer {
    int32_t variant;   // index in WRES_PK_VARIANTS
    int32_t nvirt;     // workgroups' worth of work per XCD: pixel groups x channel slices
    WresArgs w;
};

// Called by every wave of a workgroup before its first access to the layer's input: wait until all workgroups of the XCD
// have finished the previous layer, then drop this CU's L1 lines (they may hold that layer's output buffer from its use
// two layers ago). Bounded: a wait that runs out of time sets the error words and the workgroup leaves the kernel.
struct PkInputWait {
    PkCtl* ctl;
    uint32_t* s_err;      // LDS
    uint64_t deadline;    // wall clock ticks (100 MHz)
    int32_t layer;        // wait for `layer - 1` (none for 0)
    uint32_t xcd;
    uint32_t target;      // value the counter of `layer - 1` reaches when all workgroups of the XCD have arrived (thread 0)
    __device__ __forceinline__ void operator()() const {
        if (layer == 0) return;
        if (threadIdx.x == 0) {
            const uint32_t* ctr = &ctl->arrive[(xcd * kPkMaxLayers + (layer - 1)) * 16];
            // (the counters are never reset and may wrap: compare by difference)
            while ((int32_t)(__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
                __builtin_amdgcn_s_sleep(1);
                if (wall_clock64() > deadline) {
                    *s_err = 1;
                    break;
                }
            }
        }
        __syncthreads();
        asm volatile("buffer_inv sc0" ::: "memory");
    }
};

__global__ __launch_bounds__(512) void conv_wres_persistent_kernel(PkArgs p) {
    prefetch_kernel_arguments<sizeof(PkArgs)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t sWt[];
    __shared__ __attribute__((aligned(16))) uint8_t sm_raw[sizeof(WresSmemOf<4, WRES_FAST>)];  // (the largest of the variants' tables)
    __shared__ uint32_t s_err;
    // The table is read through the constant address space: it does not change while the kernel runs, and the compiler
    // may then treat its fields like kernel arguments (fetched where they are used instead of kept or spilled).

    const uint32_t xcd = blockIdx.x & 7u, rank = blockIdx.x >> 3;
    const uint32_t xcc = (uint32_t)__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15u;  // HW_REG_XCC_ID
    if (threadIdx.x == 0) s_err = xcc != xcd ? 2u : 0u;
    __syncthreads();
    const uint64_t deadline = wall_clock64() + (uint64_t)p.wait_us * 100ull;
    // The counters are not cleared between launches: every launch adds kPkPerXcd to each, so the value a counter must reach
    // follows from what this workgroup's own arrival found there (launches that share counters run one after the other,
    // and at most kPkPerXcd - 1 others can have arrived before this one).
    uint32_t target = 0;
    for (int l = 0; l < p.nlayers; ++l) {
        if (__builtin_amdgcn_readfirstlane(s_err) != 0) break;  // (uniform: read after a barrier)
        typedef const __attribute__((address_space(4))) PkLayer* table_ptr_t;
        const table_ptr_t L = (table_ptr_t)(uintptr_t)p.layers + (xcd * (uint32_t)p.nlayers + l);
        // One word of every 64-byte line of the NEXT layer's table entry is requested now and consumed after this layer:
        // the entry is then in the scalar cache when that layer starts (its fields are fetched where they are used, which
        // from memory is a chain of cold misses at the head of every layer).
        int32_t touch = 0;
        if (l + 1 < p.nlayers) {
            const __attribute__((address_space(4))) int32_t* const nl = reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(L + 1);
#pragma unroll
            for (int i = 0; i < (int)((sizeof(PkLayer) + 63) / 64); ++i) touch += nl[16 * i];
        }
        __builtin_amdgcn_sched_barrier(0);
        const int32_t variant = L->variant, nvirt = L->nvirt;
        const __attribute__((address_space(4))) WresArgs& w = L->w;
        const PkInputWait wait = {p.ctl, &s_err, deadline, l, xcd, target};
        for (uint32_t v = rank; v < (uint32_t)nvirt; v += kPkPerXcd) {
            const uint32_t slice = v / w.ngroups, group = v - slice * w.ngroups;
            switch (variant) {
#define X(ID, NF, BF, MODE, D, LM)                                                                                        \
    case ID:                                                                                                              \
        conv_wres_body<NF, BF, MODE, D, LM>(w, group, slice, sWt, *reinterpret_cast<WresSmemOf<NF, MODE>*>(sm_raw), wait); \
        break;
                WRES_PK_VARIANTS(X)
#undef X
            default: break;
            }
            __syncthreads();  // every wave has left the LDS weights and tables
        }
        // This workgroup's share of layer l is stored: count it in. Every wave first waits until the L2 has acknowledged
        // all of its own stores (vmcnt(0), said explicitly: a workgroup-scope release need not wait for them), so that once
        // the barrier below has passed, the whole workgroup's output is in the XCD's L2 before thread 0 arrives.
        asm volatile("" ::"s"(touch));       // (the words requested above are done with)
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters untouched
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t found = __hip_atomic_fetch_add(&p.ctl->arrive[(xcd * kPkMaxLayers + l) * 16], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            target = (found & ~(uint32_t)(kPkPerXcd - 1)) + kPkPerXcd;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0 && s_err != 0) {
        atomicMax(&p.ctl->error, s_err);
        // (a plain store: any non-zero code reports the failure, and a read-modify-write on host memory needs atomic
        // routing over the bus that a platform may lack)
        if (p.host_error != nullptr) __hip_atomic_store(p.host_error, s_err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// ---- fixed workspace -----------------------------------------------------------------------------------------------------
// Layout: [0, 256) the sticky error word; then the counters; then the layer tables of up to kPkMaxLayers layers.
constexpr size_t kWsCtl = 256;
constexpr size_t kWsTable = kWsCtl + (sizeof(PkCtl) + 255) / 256 * 256;
constexpr size_t kWsTableBytes = (size_t)8 * kPkMaxLayers * sizeof(PkLayer);
constexpr size_t kWsBytes = kWsTable + kWsTableBytes;   // 281 KiB on every device the library runs on
// Host code must never use this name as an address (on the host it is a stand-in, not device memory): the device
// address comes from hipGetSymbolAddress, below, and only that pointer is handed to kernels and copies.
static __device__ __align__(256) uint8_t scratch[kWsBytes];

int pk_variant_of(int tag) {
#define X(ID, NF, BF, MODE, D, LM) \
    if (tag == wres_tag(NF, BF, MODE, D, LM)) return ID;
    WRES_PK_VARIANTS(X)
#undef X
    return -1;
}

}  // namespace

hipError_t pk_workspace(int device, PkWorkspace* ws) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static uint8_t* base_of[kMaxDevices] = {};
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    int current = -1;
    if (const hipError_t e = hipGetDevice(&current); e != hipSuccess) return e;
    if (current != device) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lk(mu);
    if (base_of[device] == nullptr) {
        void* p = nullptr;
        if (const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        base_of[device] = static_cast<uint8_t*>(p);
    }
    uint8_t* const base = base_of[device];
    ws->error = reinterpret_cast<uint32_t*>(base);
    ws->ctl = reinterpret_cast<PkCtl*>(base + kWsCtl);
    ws->table = base + kWsTable;
    ws->table_bytes = kWsTableBytes;
    return hipSuccess;
}

bool wres_pk_has_variant(int tag) {
    return pk_variant_of(tag) >= 0;
}

hipError_t wres_pk_make(const std::vector<PkLayerDesc>& layers, std::vector<uint8_t>* table, RecordedLaunch* launch) {
    if (layers.empty() || (int)layers.size() > kPkMaxLayers) return hipErrorInvalidValue;
    table->assign(8 * layers.size() * sizeof(PkLayer), 0);
    size_t lds = 0;
    for (size_t i = 0; i < layers.size(); ++i) {
        const RecordedLaunch& r = *layers[i].launch;
        PkLayer L;
        memset(&L, 0, sizeof(L));
        L.variant = pk_variant_of(r.tag);
        if (L.variant < 0 || r.arg.size() * 8 < sizeof(WresArgs) || r.block.x != 512) return hipErrorNotSupported;
        memcpy(&L.w, r.arg.data(), sizeof(WresArgs));
        L.nvirt = (int32_t)(L.w.ngroups * r.grid.y);
        for (int x = 0; x < 8; ++x) {
            PkLayer Lx = L;
            Lx.w.a.in += x * layers[i].d_in;
            Lx.w.a.out += x * layers[i].d_out;
            if (Lx.w.fz.other != nullptr) Lx.w.fz.other += x * layers[i].d_other;
            if (Lx.w.fz.out != nullptr) Lx.w.fz.out += x * layers[i].d_fzout;
            memcpy(table->data() + ((size_t)x * layers.size() + i) * sizeof(PkLayer), &Lx, sizeof(Lx));
        }
        lds = std::max<size_t>(lds, r.lds);
    }
    // (at least 100 KiB of dynamic LDS: no second workgroup fits a CU, so the 256 workgroups are one per CU)
    lds = std::max<size_t>(lds, 100 * 1024);
    auto kernel = &conv_wres_persistent_kernel;
    static LdsGrant grant;
    if (const hipError_t e = grant.ensure(reinterpret_cast<const void*>(kernel), lds, 48 * 1024); e != hipSuccess) return e;
    launch->func = reinterpret_cast<const void*>(kernel);
    launch->grid = dim3(kPkWorkgroups);
    launch->block = dim3(512);
    launch->lds = (uint32_t)lds;
    launch->tag = 0;
    return hipSuccess;
}
#endif  // WRES_PART == 3

}  // namespace nce
