// Pieces shared by the convolution kernels that keep matrix operands in LDS as 1 KiB blocks of 16 rows x 64 bytes filled
// by global_load_lds_dwordx4 (16 bytes per lane from global memory straight into LDS) and read back as MFMA operands with
// ds_read_b128: the bank-conflict-free placement of a row's four 16-byte pieces, and the wait-count immediate.
#pragma once

#include <stdint.h>

namespace nce {
namespace lds_detail {

// How ds_read_b128 is served on gfx950 (measured with two lanes at a time reading one bank group at different addresses
// while every other lane reads one common address): four clocks of sixteen lanes each, and the sixteen are not
// neighbours - lanes {0-3, 12-15, 20-27}, then {4-11, 16-19, 28-31}, then the same two sets 32 higher. Within a set, lanes
// that read different addresses of the same 16-byte bank group (64 banks x 4 bytes = sixteen groups, address / 16 mod 16)
// take one more clock per extra address; every pattern timed fits that model (256 bytes/clock when the sixteen lanes of
// each set cover the sixteen groups, 128 bytes/clock for a row-per-lane pattern without the right swizzle).
//
// In the operand read of v_mfma_i32_16x16x64_i8, lane 16 q + r takes piece q (16 bytes) of row r, so a set holds every
// row exactly once: rows 0-3 and 12-15 with one piece, rows 4-11 with its neighbour q ^ 1.

// Block of 16 rows x 64 bytes: piece p of row r sits at r * 64 + ((p ^ swz(r)) << 4). Rows r, r + 4, r + 8, r + 12 share
// the bank groups 4 (r % 4) .. 4 (r % 4) + 3; with swz = 0, 3, 2, 1 for the four quarters of the rows, the pieces one set
// takes from them (q, q ^ 1, q ^ 1, q) land at four different positions.
__device__ __forceinline__ int swz(int r) {
    return (-(r >> 2)) & 3;
}

// s_waitcnt immediate that waits until at most n vector-memory operations are outstanding (nothing else).
constexpr int vmcnt_imm(int n) {
    return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14);
}

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// One global_load_lds_dwordx4: lane l's 16 bytes at `src` go to LDS at `block` + 16 l (block: uniform, a pointer into
// __shared__ memory). Written as inline assembly on purpose: in a kernel that contains the compiler's own builtin for
// this instruction, every wait the compiler inserts on the LDS counter is a wait for ALL outstanding LDS reads (it no
// longer counts them), which serialises each ds_read with its use; the assembly form leaves its counting intact. The
// transfer counts as a vector-memory operation: wait with vmcnt (vmcnt_imm) - and a barrier, for other waves - before the
// block is read. The "memory" clobber keeps the compiler from moving LDS or global accesses across the request.
__device__ __forceinline__ void load_to_lds_16(const void* src, void* block) {
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)block;
    // (m0 is named as clobbered so that the compiler does not carry a value of its own in it across the request; it warns
    // about reserved registers in clobber lists in general)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory", "m0");
#pragma clang diagnostic pop
}

}  // namespace lds_detail
}  // namespace nce
