// Host-side state shared by the kernel launchers: device properties, tuning
// knobs, HIP error capture.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mccl_hip.h"

namespace mcclhip {

struct DeviceInfo {
    int device = -1;
    int num_cus = 256;
    bool ok = false;
};

// Lazily initialised properties of the current device (mccl_hip_init).
const DeviceInfo& device_info();

struct Tuning {
    int fold_blocks_per_cu = 256;  // grid cap of the streaming kernels, in blocks per CU
    int nontemporal = 1;         // 1: streaming loads/stores carry the `nt` hint (+8..12 % on MI355X)
    int topk_path = 0;           // 0 auto, 1 multi-pass exact path only, 2 single-pass path at any size
    int topk_stall_test = 0;     // tests only: 1 = the sample blocks publish a wrong epoch, so that every wait of the single-pass path runs into its limit
    int topk_barrier_ms = 2000;  // single-pass path: longest wait of a block for another block of its launch
    int fp16_portable = 0;       // FP16 casts: 1 = the reference's portable branch (half subnormals flushed, NaN bits passed through)
    int sparse_path = 0;         // sparse accumulate with a workspace: 0 auto (runs of tiles up to 8 ranks), 1 tile kernels only
    int sparse_run_steps = 0;    // runs of tiles: 2048-element tiles per wavefront, 0 = from the input's size
};
Tuning& tuning();

void record_hip_error(hipError_t e);

#define MCCLHIP_TRY(expr)                            \
    do {                                             \
        hipError_t _e = (expr);                      \
        if (_e != hipSuccess) {                      \
            ::mcclhip::record_hip_error(_e);         \
            return MCCL_HIP_ERR_RUNTIME;             \
        }                                            \
    } while (0)

// sparse.hip: resolves the current device's copy of the static scratch array of
// mccl_hip_sparse_accumulate_static (once per device, from mccl_hip_init).
int sparse_static_setup(int device);

// Call after every kernel launch: launch-time errors surface here.
inline int launch_status() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        record_hip_error(e);
        return MCCL_HIP_ERR_RUNTIME;
    }
    return MCCL_HIP_OK;
}

inline uint32_t clamp_u32(uint64_t v, uint64_t lo, uint64_t hi) {
    return (uint32_t)(v < lo ? lo : (v > hi ? hi : v));
}

}  // namespace mcclhip
