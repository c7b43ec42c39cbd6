// Persistent segments of a task list: consecutive convolutions (with their fused residual adds) of the weights-resident
// kernels run as ONE launch of 256 workgroups, one per CU, that walk the layers themselves.
//
// What makes that cheap on MI355X: the eight XCDs have private L2 caches that are coherent only through memory, but
// within an XCD the 32 CUs share one L2. A segment therefore gives XCD x the images [x * N/8, (x + 1) * N/8) of EVERY
// layer: whatever a layer reads was written by the same XCD (or before the launch), so the dependency between two layers
// is a barrier among the 32 workgroups of an XCD - stores waited for, an arrival counter per XCD and layer, an L1
// invalidate - with no L2 write-back or invalidate. The next layer's weights are requested before that wait.
#pragma once

#include "nce_common.h"

#include <vector>

namespace nce {

constexpr int kPkMaxLayers = 64;
constexpr int kPkWorkgroups = 256;   // one per CU; workgroup b runs on XCD b % 8 (checked by the kernel)
constexpr int kPkPerXcd = 32;

struct PkCtl {
    uint32_t error;                            // 1: a wait ran out of time, 2: a workgroup found itself on an unexpected XCD
    uint32_t pad[15];
    uint32_t arrive[8 * kPkMaxLayers * 16];    // [xcd][layer], one 64-byte line per counter; multiples of 32 between launches
};

struct PkArgs {
    const void* layers;     // device table made by wres_pk_make
    PkCtl* ctl;             // counters: zero when first used, then only ever counted up (by 32 per launch and counter)
    uint32_t* host_error;   // host-visible word that receives ctl->error (may be null)
    int32_t nlayers;
    uint32_t wait_us;       // from the kernel's start; a wait still unsatisfied then gives up and the workgroup leaves
};

// One layer of a segment as recorded in per-XCD form, and the byte offsets of an XCD's share of its tensors.
struct PkLayerDesc {
    const RecordedLaunch* launch;
    int64_t d_in, d_out, d_other, d_fzout;
};

// The library's fixed workspace on a device: what a segment otherwise gets from hipMalloc, for the enqueue form that
// allocates nothing. One per device and process, shared by every list that uses that form.
struct PkWorkspace {
    uint32_t* error = nullptr;   // sticky error word (device memory): raised by a segment that gave up, cleared by the host
    PkCtl* ctl = nullptr;        // counters (zero at load; zeroed again by the host after a launch that gave up)
    uint8_t* table = nullptr;    // layer tables of the list that is running
    size_t table_bytes = 0;      // room for the tables of kPkMaxLayers layers
};
// Looks the workspace's device address up (once per device, cached). `device` must be the calling thread's current device.
hipError_t pk_workspace(int device, PkWorkspace* ws);

bool wres_pk_has_variant(int tag);
// The device table of a segment (to be uploaded) and its launch: kernel, grid, block, LDS size; the argument block
// (PkArgs) is filled in by the caller once the table and counters have device addresses.
hipError_t wres_pk_make(const std::vector<PkLayerDesc>& layers, std::vector<uint8_t>* table, RecordedLaunch* launch);

}  // namespace nce
