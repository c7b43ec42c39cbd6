// Internal declarations shared by the host side (nce_api.cpp) and the kernel files.
#pragma once

#include <atomic>
#include <cstring>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <vector>

#include "../../include/nce_hip.h"
#include "nce_log.h"

namespace nce {

// Epilogue parameters in the form the kernels consume. The host folds the descriptor's clamp
// domain, the output zero point and the storage range of the output type into one clamp that is
// applied BEFORE the zero point is added: y = med3(y, lo, hi) + zp. With L <= H this is identical
// to "add zp, clamp to [L, H], saturate to the type" because every bound stays far inside int32.
struct PpeDev {
    int32_t lo, hi;        // clamp in the zero-point-free domain
    int32_t zp_out;        // output zero point (0 for MAXPOOL)
    int32_t prelu_mult;    // multiplier for negative values (1,0 = identity; 0,0 = ReLU)
    int32_t prelu_shift;
    int32_t round_mode;    // nce_round_mode_t
    int32_t quant_mult;    // scale when there is no weight table (ELTWISE / AVEPOOL)
    int32_t quant_shift;
    int32_t in1_mult, in2_mult;  // ELTWISE per-input multipliers (1,1 when absent)
};

// An output sub-box (one DPUTask variant, or the whole tensor) in output coordinates.
struct Box {
    int32_t x0, y0, z0;  // inclusive start
    int32_t bw, bh, bc;  // extent in x (W), y (H), z (C)
};

struct TensorDev {
    uint8_t* data;
    int64_t sn, sh, sw;  // strides in bytes for N, H, W
    int64_t sc;          // channel stride: 1 (NHWC) except for outputs in a permuted order (ODU permutation)
    int32_t n, c, h, w;
    int32_t is_signed;   // storage type i8
    int32_t zp;
};

struct TaskDev {
    TensorDev in, in2, out;  // in2: second eltwise input
    const uint8_t* weights;
    int64_t w_stride_oc;     // bytes between weight sets (conv) / per-channel rows (depthwise)
    int32_t w_is_signed, w_zp;
    const int32_t* table;    // weight table rows of 4 x int32, or nullptr
    int64_t table_stride;    // int32 elements between rows
    int32_t ky, kx, sy, sx, pt, pl, pr;
    PpeDev ppe;
};

// MI355X spreads consecutive workgroup ids over its 8 XCDs (id % 8), each with a private L2. Tiles that
// share input rows should share an L2, so kernels walk their tiles in this order: XCD x gets the
// contiguous range [x * per_xcd, (x + 1) * per_xcd). Launch 8 * per_xcd workgroups, per_xcd =
// ceil(ntiles / 8); ids mapped at or beyond ntiles have nothing to do.
constexpr int kNumXcd = 8;
__host__ __device__ inline uint32_t xcd_grid(uint32_t ntiles) {
    return kNumXcd * ((ntiles + kNumXcd - 1) / kNumXcd);
}
__device__ inline uint32_t xcd_tile(uint32_t block_id, uint32_t ntiles) {
    const uint32_t per_xcd = (ntiles + kNumXcd - 1) / kNumXcd;
    return (block_id % kNumXcd) * per_xcd + block_id / kNumXcd;
}

// Kernel arguments sit in memory and reach the scalar registers through scalar loads that the compiler places next to
// their first use: a kernel with a few hundred bytes of arguments then starts with a CHAIN of cold misses, one per group
// of 64-byte lines it touches for the first time (four in the weights-resident convolution: 0.3-0.7 us each from memory,
// with a wait between them). Called first thing in a kernel, this requests one word of every line of the argument block
// at once and waits for them together; the compiler's own loads then find the lines in the scalar cache.
// BYTES = sizeof of the kernel's argument struct (its only parameter).
template <int BYTES>
__device__ __forceinline__ void prefetch_kernel_arguments() {
#ifdef __HIP_DEVICE_COMPILE__
    constexpr int LINES = (BYTES + 63) / 64;
    static_assert(LINES >= 1 && LINES <= 16, "argument block larger than this helper covers");
    const auto p = __builtin_amdgcn_kernarg_segment_ptr();  // (constant address space)
    // (one statement: the loaded words are thrown away, and a register the compiler took back before the word arrived
    // would be overwritten later)
    int t[16];
#define NCE_KA_LOAD(i) "s_load_dword %" #i ", %16, " #i "*64\n\t"
    if constexpr (LINES <= 4) {
        asm volatile(NCE_KA_LOAD(0) NCE_KA_LOAD(1) NCE_KA_LOAD(2) NCE_KA_LOAD(3) "s_waitcnt lgkmcnt(0)"
                     : "=s"(t[0]), "=s"(t[1]), "=s"(t[2]), "=s"(t[3]), "=s"(t[4]), "=s"(t[5]), "=s"(t[6]), "=s"(t[7]), "=s"(t[8]), "=s"(t[9]), "=s"(t[10]),
                       "=s"(t[11]), "=s"(t[12]), "=s"(t[13]), "=s"(t[14]), "=s"(t[15])
                     : "s"(p));
    } else if constexpr (LINES <= 8) {
        asm volatile(NCE_KA_LOAD(0) NCE_KA_LOAD(1) NCE_KA_LOAD(2) NCE_KA_LOAD(3) NCE_KA_LOAD(4) NCE_KA_LOAD(5) NCE_KA_LOAD(6) NCE_KA_LOAD(7) "s_waitcnt lgkmcnt(0)"
                     : "=s"(t[0]), "=s"(t[1]), "=s"(t[2]), "=s"(t[3]), "=s"(t[4]), "=s"(t[5]), "=s"(t[6]), "=s"(t[7]), "=s"(t[8]), "=s"(t[9]), "=s"(t[10]),
                       "=s"(t[11]), "=s"(t[12]), "=s"(t[13]), "=s"(t[14]), "=s"(t[15])
                     : "s"(p));
    } else if constexpr (LINES <= 12) {
        asm volatile(NCE_KA_LOAD(0) NCE_KA_LOAD(1) NCE_KA_LOAD(2) NCE_KA_LOAD(3) NCE_KA_LOAD(4) NCE_KA_LOAD(5) NCE_KA_LOAD(6) NCE_KA_LOAD(7) NCE_KA_LOAD(8)
                     NCE_KA_LOAD(9) NCE_KA_LOAD(10) NCE_KA_LOAD(11) "s_waitcnt lgkmcnt(0)"
                     : "=s"(t[0]), "=s"(t[1]), "=s"(t[2]), "=s"(t[3]), "=s"(t[4]), "=s"(t[5]), "=s"(t[6]), "=s"(t[7]), "=s"(t[8]), "=s"(t[9]), "=s"(t[10]),
                       "=s"(t[11]), "=s"(t[12]), "=s"(t[13]), "=s"(t[14]), "=s"(t[15])
                     : "s"(p));
    } else {
        asm volatile(NCE_KA_LOAD(0) NCE_KA_LOAD(1) NCE_KA_LOAD(2) NCE_KA_LOAD(3) NCE_KA_LOAD(4) NCE_KA_LOAD(5) NCE_KA_LOAD(6) NCE_KA_LOAD(7) NCE_KA_LOAD(8)
                     NCE_KA_LOAD(9) NCE_KA_LOAD(10) NCE_KA_LOAD(11) NCE_KA_LOAD(12) NCE_KA_LOAD(13) NCE_KA_LOAD(14) NCE_KA_LOAD(15) "s_waitcnt lgkmcnt(0)"
                     : "=s"(t[0]), "=s"(t[1]), "=s"(t[2]), "=s"(t[3]), "=s"(t[4]), "=s"(t[5]), "=s"(t[6]), "=s"(t[7]), "=s"(t[8]), "=s"(t[9]), "=s"(t[10]),
                       "=s"(t[11]), "=s"(t[12]), "=s"(t[13]), "=s"(t[14]), "=s"(t[15])
                     : "s"(p));
    }
#undef NCE_KA_LOAD
    __builtin_amdgcn_sched_barrier(0);  // (nothing that follows - in particular no argument load with its own wait - moves ahead of the requests)
#endif
}

// Store 16 (or 8) consecutive channels of one pixel: one vector store when channels are compact, byte
// stores at the channel stride for permuted output orders. p points at the first of those channels.
__device__ __forceinline__ void store_channels16(uint8_t* p, int64_t sc, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
    if (sc == 1) {
        *reinterpret_cast<uint4*>(p) = make_uint4(w0, w1, w2, w3);
    } else {
        const uint32_t w[4] = {w0, w1, w2, w3};
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i * sc] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
    }
}
__device__ __forceinline__ void store_channels8(uint8_t* p, int64_t sc, uint32_t w0, uint32_t w1) {
    if (sc == 1) {
        *reinterpret_cast<uint2*>(p) = make_uint2(w0, w1);
    } else {
        const uint32_t w[2] = {w0, w1};
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i * sc] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
    }
}

// Opt a kernel in to `bytes` of dynamic LDS. The runtime call is made only when a launch needs more than
// what this kernel was already granted on the current device, so steady-state launches make no runtime
// call besides the launch itself. One LdsGrant per kernel instantiation (a function-local static).
struct LdsGrant {
    static constexpr int kMaxDevices = 64;
    std::atomic<size_t> granted[kMaxDevices];
    LdsGrant() {
        for (auto& g : granted) g.store(0, std::memory_order_relaxed);
    }
    hipError_t ensure(const void* kernel, size_t bytes, size_t default_limit) {
        if (bytes <= default_limit) return hipSuccess;
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < kMaxDevices && granted[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < kMaxDevices) {
            size_t cur = granted[dev].load(std::memory_order_relaxed);
            while (cur < bytes && !granted[dev].compare_exchange_weak(cur, bytes, std::memory_order_release)) {
            }
        }
        return hipSuccess;
    }
};

// Tuning / test knobs of an executor. Read from the environment ONCE, when the executor is created
// (nceExecutorCreate); a launch never calls getenv.
struct Options {
    int conv_path = 0;        // NCE_HIP_CONV_PATH: 1 = skip the weights-resident kernel, 2 = gather kernel only
    bool wres_forced = false; // NCE_HIP_CONV_WRES="nf,bf,nwaves,tiles_per_wave" was given ...
    int wres[4] = {0, 0, 0, 0};  // ... with these values
    int halo_tile = -1;       // NCE_HIP_CONV_TILE: force one halo tile shape (0..3)
    bool no_fuse = false;     // NCE_HIP_NO_FUSE: task lists never run a convolution and the add after it as one launch
    int persistent = 0;       // NCE_HIP_PERSISTENT: task lists run runs of weights-resident convolutions as one persistent launch
    int persistent_wait_us = 2000000;  // NCE_HIP_PERSISTENT_WAIT_US: time after which a persistent launch's waits give up
    int tiled = -1;           // NCE_HIP_CONV_TILED: -1 automatic, 0 never, 1.. force that shape of the LDS-tiled kernel
    int patch = -1;           // NCE_HIP_CONV_PATCH: -1 automatic, 0 never, 1 = wherever its conditions hold; "nf,pr[,waves]" also forces its shape
    int patch_nf = 0, patch_pr = 0, patch_waves = 0, patch_npx = 0;
    bool env_path = false;    // NCE_HIP_CONV_PATH was given at all (switches the conv + add fusion off, as NO_FUSE does)
};

// One prepared kernel launch: the kernel, its grid and a copy of its (single, by-value) argument struct.
struct RecordedLaunch {
    const void* func = nullptr;
    dim3 grid, block;
    uint32_t lds = 0;
    std::vector<uint64_t> arg;  // argument bytes (8-byte aligned storage; the largest member of every argument struct is 8 bytes)
    int32_t tag = 0;            // weights-resident convolution kernels: their template parameters, packed (else 0)
};

// What a launch_* function needs besides its task: the executor's options and, when a task list prepares its
// launches, the list to record into instead of launching. Set by the C-ABI entry points around their calls
// (thread-local: one executor may be used from several host threads).
struct LaunchContext {
    const Options* opt = nullptr;
    std::vector<RecordedLaunch>* record = nullptr;
    nce_log_s* log = nullptr;   // the executor's log (kernel choices are noted there at level 3)
    // Per-XCD form: the task is one eighth of the batch, to be run by the 32 CUs of one XCD inside a persistent segment
    // (grids are sized for 32 CUs; only the weights-resident convolution kernels take part).
    bool per_xcd = false;
};
extern thread_local LaunchContext tls_launch;
inline const Options& options() {
    static const Options defaults;
    return tls_launch.opt ? *tls_launch.opt : defaults;
}

// Launch `kernel(arg)` now, or record the launch when a task list is being prepared.
template <typename Arg>
inline hipError_t emit(void (*kernel)(Arg), dim3 grid, dim3 block, size_t lds, hipStream_t stream, const Arg& arg, int tag = 0) {
    if (std::vector<RecordedLaunch>* rec = tls_launch.record) {
        RecordedLaunch r;
        r.tag = tag;
        r.func = reinterpret_cast<const void*>(kernel);
        r.grid = grid;
        r.block = block;
        r.lds = (uint32_t)lds;
        r.arg.resize((sizeof(Arg) + 7) / 8);
        memcpy(r.arg.data(), &arg, sizeof(Arg));
        rec->push_back(std::move(r));
        return hipSuccess;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, arg);
    return hipGetLastError();
}
inline hipError_t replay(const RecordedLaunch& r, hipStream_t stream) {
    void* args[1] = {const_cast<uint64_t*>(r.arg.data())};
    return hipLaunchKernel(r.func, r.grid, r.block, args, r.lds, stream);
}

hipError_t launch_eltwise(const TaskDev& t, const Box& box, hipStream_t stream);
hipError_t launch_pool(const TaskDev& t, const Box& box, bool is_max, hipStream_t stream);
hipError_t launch_dwconv(const TaskDev& t, const Box& box, hipStream_t stream);
hipError_t launch_conv(const TaskDev& t, const Box& box, hipStream_t stream);
// The convolution `conv` and the ELTWISE task `add` that directly follows it in a task list as ONE launch, when the add
// reads the convolution's output and everything else allows it; hipErrorNotSupported (nothing launched) otherwise.
hipError_t launch_conv_fused_add(const TaskDev& conv, const Box& conv_box, const TaskDev& add, const Box& add_box, hipStream_t stream);
struct FuseAdd;
// Integer constants of a uniform-scale ELTWISE add whose first input is `first_is_other ? other : produced`; false when
// the task needs another arithmetic path.
bool eltwise_fuse_params(const TaskDev& add, bool produced_is_in1, FuseAdd* out);

}  // namespace nce
