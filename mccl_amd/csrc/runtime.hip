// Library state, error text, tuning knobs and the stream-ordering (fence) API.
//
// The reference orders its kernel queue against consumers with three
// MTLSharedEvents and monotonically increasing values
// (csrc/metal/EventSync.mm:19-30,:189-206).  Here a fence ticket is the index
// of a hipEvent recorded on the caller's stream; events live in a fixed ring.
#include "runtime.h"

#include <atomic>
#include <chrono>
#include <cstring>
#include <mutex>
#include <thread>

namespace mcclhip {

namespace {
std::mutex g_mu;        // device properties, tuning
std::mutex g_fence_mu;  // the fence ring: never held across a wait for the device
DeviceInfo g_info;
Tuning g_tuning;
thread_local int t_last_hip_error = 0;

constexpr uint64_t kRing = 1024;
constexpr int kMaxFenceDevices = 64;
// One ring of events per device, created on first use and never destroyed (a
// waiter may be polling an event outside the lock).  Slot s is owned by the
// newest ticket t with t % kRing == s; g_slot_ticket names it, g_slot_device
// the device whose ring holds its event.
hipEvent_t* g_ring[kMaxFenceDevices];
uint64_t g_slot_ticket[kRing];
int g_slot_device[kRing];
std::atomic<uint64_t> g_next_ticket{1};
}  // namespace

void record_hip_error(hipError_t e) { t_last_hip_error = (int)e; }

const DeviceInfo& device_info() { return g_info; }
Tuning& tuning() { return g_tuning; }

}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

int mccl_hip_abi_version(void) { return MCCL_HIP_ABI_VERSION; }

int mccl_hip_init(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    int dev = -1;
    MCCLHIP_TRY(hipGetDevice(&dev));
    if (g_info.ok && g_info.device == dev) return MCCL_HIP_OK;
    hipDeviceProp_t prop;
    MCCLHIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        // Code objects in this library exist for gfx950 only.
        record_hip_error(hipErrorNoBinaryForGpu);
        return MCCL_HIP_ERR_RUNTIME;
    }
    int rc = sparse_static_setup(dev);
    if (rc) return rc;
    g_info.device = dev;
    g_info.num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    g_info.ok = true;
    return MCCL_HIP_OK;
}

const char* mccl_hip_strerror(int code) {
    switch (code) {
        case MCCL_HIP_OK: return "ok";
        case MCCL_HIP_ERR_OP: return "Unsupported ReduceOp";
        case MCCL_HIP_ERR_DTYPE: return "unsupported element type";
        case MCCL_HIP_ERR_CAPACITY: return "TopK compress: buffer too small";
        case MCCL_HIP_ERR_SIZE: return "TopK decompress: size mismatch";
        case MCCL_HIP_ERR_INDEX: return "TopK decompress: index out of bounds";
        case MCCL_HIP_ERR_ARG: return "invalid argument";
        case MCCL_HIP_ERR_RUNTIME: return "HIP runtime call failed";
        case MCCL_HIP_ERR_WORKSPACE: return "workspace too small";
        case MCCL_HIP_ERR_TIMEOUT: return "fence wait timed out";
        case MCCL_HIP_ERR_POINTER: return "pointer is not GPU-accessible memory";
        default: return "unknown error";
    }
}

int mccl_hip_last_hip_error(void) { return t_last_hip_error; }

int mccl_hip_pointer_check(const void* ptr, uint64_t nbytes, void** device_ptr) {
    if (!ptr || !device_ptr) return MCCL_HIP_ERR_ARG;
    int dev = -1;
    MCCLHIP_TRY(hipGetDevice(&dev));
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, ptr);
    if (e == hipErrorInvalidValue) {  // how older runtimes report memory they do not know
        (void)hipGetLastError();
        return MCCL_HIP_ERR_POINTER;
    }
    if (e != hipSuccess) {
        record_hip_error(e);
        (void)hipGetLastError();
        return MCCL_HIP_ERR_RUNTIME;
    }
    void* dp = nullptr;
    switch (attr.type) {
        case hipMemoryTypeDevice: {
            if (attr.device != dev) return MCCL_HIP_ERR_POINTER;
            hipDeviceptr_t base = nullptr;
            size_t size = 0;
            e = hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return MCCL_HIP_ERR_POINTER;
            }
            const uintptr_t lo = (uintptr_t)base, p = (uintptr_t)ptr;
            if (p < lo || nbytes > size || p - lo > size - nbytes) return MCCL_HIP_ERR_POINTER;
            dp = const_cast<void*>(ptr);
            break;
        }
        case hipMemoryTypeManaged:
        case hipMemoryTypeHost: {  // pinned: kernels reach it through its device-side alias
            dp = attr.type == hipMemoryTypeHost ? attr.devicePointer : const_cast<void*>(ptr);
            if (!dp) return MCCL_HIP_ERR_POINTER;
            // the whole range must lie inside the allocation, as for device memory; an extent
            // that cannot be determined is not vouched for
            hipDeviceptr_t base = nullptr;
            size_t size = 0;
            uintptr_t p = (uintptr_t)ptr;
            e = hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr);
            if (e != hipSuccess && dp != ptr) {
                (void)hipGetLastError();
                p = (uintptr_t)dp;
                e = hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)dp);
            }
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return MCCL_HIP_ERR_POINTER;
            }
            const uintptr_t lo = (uintptr_t)base;
            if (p < lo || nbytes > size || p - lo > size - nbytes) return MCCL_HIP_ERR_POINTER;
            break;
        }
        default:
            return MCCL_HIP_ERR_POINTER;
    }
    *device_ptr = dp;
    return MCCL_HIP_OK;
}

int mccl_hip_set_tuning(const char* key, int value) {
    if (!key) return MCCL_HIP_ERR_ARG;
    Tuning& t = tuning();
    if (!std::strcmp(key, "fold_blocks_per_cu")) {
        if (value < 1 || value > 4096) return MCCL_HIP_ERR_ARG;
        t.fold_blocks_per_cu = value;
    } else if (!std::strcmp(key, "nontemporal")) {
        t.nontemporal = value ? 1 : 0;
    } else if (!std::strcmp(key, "topk_path")) {
        if (value < 0 || value > 2) return MCCL_HIP_ERR_ARG;
        t.topk_path = value;
    } else if (!std::strcmp(key, "topk_stall_test")) {
        t.topk_stall_test = value ? 1 : 0;
    } else if (!std::strcmp(key, "topk_barrier_ms")) {
        if (value < 0 || value > 60000) return MCCL_HIP_ERR_ARG;
        t.topk_barrier_ms = value;
    } else if (!std::strcmp(key, "fp16_portable")) {
        t.fp16_portable = value ? 1 : 0;
    } else if (!std::strcmp(key, "sparse_path")) {
        if (value < 0 || value > 1) return MCCL_HIP_ERR_ARG;
        t.sparse_path = value;
    } else if (!std::strcmp(key, "sparse_run_steps")) {
        if (value < 0 || value > (1 << 20)) return MCCL_HIP_ERR_ARG;
        t.sparse_run_steps = value;
    } else {
        return MCCL_HIP_ERR_ARG;
    }
    return MCCL_HIP_OK;
}

int mccl_hip_get_tuning(const char* key) {
    if (!key) return MCCL_HIP_ERR_ARG;
    const Tuning& t = tuning();
    if (!std::strcmp(key, "fold_blocks_per_cu")) return t.fold_blocks_per_cu;
    if (!std::strcmp(key, "nontemporal")) return t.nontemporal;
    if (!std::strcmp(key, "topk_path")) return t.topk_path;
    if (!std::strcmp(key, "topk_stall_test")) return t.topk_stall_test;
    if (!std::strcmp(key, "topk_barrier_ms")) return t.topk_barrier_ms;
    if (!std::strcmp(key, "fp16_portable")) return t.fp16_portable;
    if (!std::strcmp(key, "sparse_path")) return t.sparse_path;
    if (!std::strcmp(key, "sparse_run_steps")) return t.sparse_run_steps;
    return MCCL_HIP_ERR_ARG;
}

// ---- fences ------------------------------------------------------------------

int mccl_hip_fence_signal(void* stream, uint64_t* ticket) {
    if (!ticket) return MCCL_HIP_ERR_ARG;
    int dev = -1;
    MCCLHIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxFenceDevices) return MCCL_HIP_ERR_ARG;
    for (;;) {
        hipEvent_t old = nullptr;
        {
            std::lock_guard<std::mutex> lock(g_fence_mu);
            if (!g_ring[dev]) {
                hipEvent_t* ring = new hipEvent_t[kRing];
                for (uint64_t i = 0; i < kRing; i++) {
                    hipError_t e = hipEventCreateWithFlags(&ring[i], hipEventDisableTiming);
                    if (e != hipSuccess) {
                        record_hip_error(e);
                        for (uint64_t j = 0; j < i; j++) (void)hipEventDestroy(ring[j]);
                        delete[] ring;
                        return MCCL_HIP_ERR_RUNTIME;
                    }
                }
                g_ring[dev] = ring;
            }
            const uint64_t t = g_next_ticket.load();
            const uint64_t slot = t % kRing;
            // The slot's previous owner (kRing tickets older) leaves the ring here.  "Left the
            // ring" has to mean "complete" for every later wait on it; with per-step fences that
            // are waited on promptly it already is.
            hipError_t e = hipSuccess;
            if (g_slot_ticket[slot] != 0) {
                old = g_ring[g_slot_device[slot]][slot];
                e = hipEventQuery(old);
            }
            if (e == hipSuccess) {
                MCCLHIP_TRY(hipEventRecord(g_ring[dev][slot], (hipStream_t)stream));
                g_slot_ticket[slot] = t;
                g_slot_device[slot] = dev;
                g_next_ticket.store(t + 1);
                *ticket = t;
                return MCCL_HIP_OK;
            }
            if (e != hipErrorNotReady) {
                record_hip_error(e);
                return MCCL_HIP_ERR_RUNTIME;
            }
        }
        // The old owner is still running: wait for it WITHOUT the lock (other threads' signals,
        // queries and stream waits go on meanwhile; the old owner's stream may itself be waiting
        // for work another thread has yet to enqueue through this library), then look again:
        // the ticket counter may have moved on to another slot.
        hipError_t e = hipEventSynchronize(old);
        if (e != hipSuccess) {
            record_hip_error(e);
            return MCCL_HIP_ERR_RUNTIME;
        }
    }
}

// 1 complete, 0 pending (then *ev is the ticket's event), negative on error.  A
// ticket whose slot has a newer owner was drained when that owner took the slot.
static int fence_state_locked(uint64_t ticket, hipEvent_t* ev) {
    if (ticket == 0) return 1;
    if (ticket >= g_next_ticket.load()) return MCCL_HIP_ERR_ARG;
    const uint64_t slot = ticket % kRing;
    if (g_slot_ticket[slot] != ticket) return 1;
    *ev = g_ring[g_slot_device[slot]][slot];
    return 0;
}
// For host-side polling outside the lock: should the slot change owner while the
// caller polls, the event then reports the newer ticket, recorded only after
// this one had completed, so the caller still never returns early.
static int fence_state(uint64_t ticket, hipEvent_t* ev) {
    std::lock_guard<std::mutex> lock(g_fence_mu);
    return fence_state_locked(ticket, ev);
}

int mccl_hip_fence_query(uint64_t ticket) {
    hipEvent_t ev;
    int st = fence_state(ticket, &ev);
    if (st != 0) return st;
    hipError_t e = hipEventQuery(ev);
    if (e == hipSuccess) return 1;
    if (e == hipErrorNotReady) return 0;
    record_hip_error(e);
    return MCCL_HIP_ERR_RUNTIME;
}

int mccl_hip_fence_wait(uint64_t ticket, int timeout_ms) {
    hipEvent_t ev;
    int st = fence_state(ticket, &ev);
    if (st < 0) return st;
    if (st == 1) return MCCL_HIP_OK;
    const auto limit = std::chrono::milliseconds(timeout_ms > 0 ? timeout_ms : 30000);
    const auto start = std::chrono::steady_clock::now();
    int spins = 0;
    for (;;) {
        hipError_t e = hipEventQuery(ev);
        if (e == hipSuccess) return MCCL_HIP_OK;
        if (e != hipErrorNotReady) {
            record_hip_error(e);
            return MCCL_HIP_ERR_RUNTIME;
        }
        if (std::chrono::steady_clock::now() - start > limit) return MCCL_HIP_ERR_TIMEOUT;
        if (++spins > 2000) std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}

int mccl_hip_fence_block_stream(uint64_t ticket, void* stream) {
    // under the lock: the wait must be enqueued on this ticket's record, not on a
    // later record of the same event
    std::lock_guard<std::mutex> lock(g_fence_mu);
    hipEvent_t ev;
    int st = fence_state_locked(ticket, &ev);
    if (st < 0) return st;
    if (st == 1) return MCCL_HIP_OK;
    MCCLHIP_TRY(hipStreamWaitEvent((hipStream_t)stream, ev, 0));
    return MCCL_HIP_OK;
}

int mccl_hip_sync(void* stream) {
    MCCLHIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return MCCL_HIP_OK;
}

}  // extern "C"
