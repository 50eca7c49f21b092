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
std::mutex g_mu;
DeviceInfo g_info;
Tuning g_tuning;
thread_local int t_last_hip_error = 0;

constexpr uint64_t kRing = 1024;
hipEvent_t g_events[kRing];
bool g_event_made[kRing];
int g_event_device[kRing];
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
        default: return "unknown error";
    }
}

int mccl_hip_last_hip_error(void) { return t_last_hip_error; }

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
    return MCCL_HIP_ERR_ARG;
}

// ---- fences ------------------------------------------------------------------

int mccl_hip_fence_signal(void* stream, uint64_t* ticket) {
    if (!ticket) return MCCL_HIP_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_mu);
    int dev = -1;
    MCCLHIP_TRY(hipGetDevice(&dev));
    uint64_t t = g_next_ticket.fetch_add(1);
    uint64_t slot = t % kRing;
    if (g_event_made[slot] && g_event_device[slot] != dev) {
        MCCLHIP_TRY(hipEventDestroy(g_events[slot]));
        g_event_made[slot] = false;
    }
    if (!g_event_made[slot]) {
        MCCLHIP_TRY(hipEventCreateWithFlags(&g_events[slot], hipEventDisableTiming));
        g_event_made[slot] = true;
        g_event_device[slot] = dev;
    }
    MCCLHIP_TRY(hipEventRecord(g_events[slot], (hipStream_t)stream));
    *ticket = t;
    return MCCL_HIP_OK;
}

// 1 complete, 0 pending.  A ticket that has left the ring was signalled at
// least kRing signals ago on an in-order stream of recorded events; its slot
// now belongs to a newer ticket, whose completion is awaited instead (a
// superset of what the caller asked for only when streams differ; tickets are
// meant to be waited on promptly, as in the reference's per-step fences).
static int fence_state(uint64_t ticket, hipEvent_t* ev) {
    if (ticket == 0) return 1;
    std::lock_guard<std::mutex> lock(g_mu);
    uint64_t next = g_next_ticket.load();
    if (ticket >= next) return MCCL_HIP_ERR_ARG;
    uint64_t slot = ticket % kRing;
    if (!g_event_made[slot]) return 1;
    *ev = g_events[slot];
    return 0;
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
    hipEvent_t ev;
    int st = fence_state(ticket, &ev);
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
