// Version, status strings, window layout, profiler calibration copy.

#include <atomic>
#include <climits>
#include <mutex>

#include "nanoep_device.h"

namespace nanoep {

thread_local hipError_t g_last_hip_error = hipSuccess;

namespace {

// The switches by name (behind the NANOEP_ prefix in the environment), where they sit in Tuning, and
// their process-wide values.
struct SwitchSlot {
    const char* name;
    int Tuning::*field;
};

constexpr SwitchSlot kSwitches[] = {
    {"CHUNKS_PER_BLOCK", &Tuning::chunks_per_block}, {"ROWS_PER_BLOCK", &Tuning::rows_per_block},
    {"DISPATCH_ORDER", &Tuning::dispatch_order},     {"DISPATCH_SPAN", &Tuning::dispatch_span},
    {"DISPATCH_SIDE", &Tuning::dispatch_side},       {"DISPATCH_WHOLE_ROWS", &Tuning::dispatch_whole_rows},
    {"LAYOUT_LAUNCHES", &Tuning::layout_launches},   {"WINDOW_TOKENS", &Tuning::window_tokens},
    {"RECALL_ORDER", &Tuning::recall_order},         {"FRESH_OUTPUTS", &Tuning::fresh_outputs},
    {"REBUILD_ORDER", &Tuning::rebuild_order},       {"XCDS", &Tuning::xcds},
    {"L2_BYTES", &Tuning::l2_bytes},
};
constexpr int kSwitchCount = sizeof(kSwitches) / sizeof(kSwitches[0]);

std::atomic<int> g_switch_values[kSwitchCount];
std::once_flag g_switches_once;

// NANOEP_<NAME>=<number> in the environment; unset or empty leaves the default.
void load_switches_from_environment() {
    const Tuning defaults;
    for (int i = 0; i < kSwitchCount; ++i) {
        char variable[64];
        std::snprintf(variable, sizeof(variable), "NANOEP_%s", kSwitches[i].name);
        const char* text = std::getenv(variable);
        g_switch_values[i].store(text != nullptr && *text != '\0' ? std::atoi(text) : defaults.*(kSwitches[i].field),
                                 std::memory_order_relaxed);
    }
}

int find_switch(const char* name) {
    if (name == nullptr)
        return -1;
    for (int i = 0; i < kSwitchCount; ++i)
        if (std::strcmp(name, kSwitches[i].name) == 0)
            return i;
    return -1;
}

constexpr int kMaxDevices = 64;
std::mutex g_topology_mutex;
bool g_topology_known[kMaxDevices] = {};
Topology g_topology[kMaxDevices];

}  // namespace

Tuning current_tuning() {
    std::call_once(g_switches_once, load_switches_from_environment);
    Tuning tuning;
    for (int i = 0; i < kSwitchCount; ++i)
        tuning.*(kSwitches[i].field) = g_switch_values[i].load(std::memory_order_relaxed);
    return tuning;
}

Topology current_topology(const Tuning& tuning) {
    Topology topology;  // the MI355X's numbers, for a process without a device
    int device = -1;
    if (hipGetDevice(&device) == hipSuccess && device >= 0 && device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_topology_mutex);
        if (!g_topology_known[device]) {
            Topology asked;
            int value = 0;
            if (hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && value > 0)
                asked.cus = value;
            if (hipDeviceGetAttribute(&value, hipDeviceAttributeNumberOfXccs, device) == hipSuccess && value > 0)
                asked.xcds = value;
            // the runtime reports the L2 of one XCD; a part that reports none keeps the default
            if (hipDeviceGetAttribute(&value, hipDeviceAttributeL2CacheSize, device) == hipSuccess && value >= (1 << 20))
                asked.l2_bytes = value;
            g_topology[device] = asked;
            g_topology_known[device] = true;
        }
        topology = g_topology[device];
    } else {
        (void)hipGetLastError();  // no device: not an error of the caller's
    }
    if (tuning.xcds > 0)
        topology.xcds = tuning.xcds;
    if (tuning.l2_bytes > 0)
        topology.l2_bytes = tuning.l2_bytes;
    return topology;
}

namespace {

__global__ void __launch_bounds__(kBlockThreads) copy_vectors_kernel(const u32x4* __restrict__ src,
                                                                    u32x4* __restrict__ dst,
                                                                    size_t vectors) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < vectors)
        dst[i] = src[i];
}

}  // namespace
}  // namespace nanoep

using namespace nanoep;

extern "C" {

int nanoep_abi_version(void) { return 4; }

const char* nanoep_status_string(int status) {
    switch (status) {
        case NANOEP_OK:
            return "ok";
        case NANOEP_ERR_INVALID_ARGUMENT:
            return "invalid argument";
        case NANOEP_ERR_HIP:
            return "HIP runtime error";
        case NANOEP_ERR_WORKSPACE:
            return "layout workspace too small";
        case NANOEP_ERR_TIMEOUT:
            return "timed out waiting for the layout counts";
        case NANOEP_ERR_ROUTING:
            return "routing ids must be -1 or distinct expert ids in [0, num_local_experts)";
        case NANOEP_ERR_SCRATCH_LIMIT:
            return "routing geometry needs more layout workspace than the static scratch of nanoep_layout_static holds (4 MiB)";
        default:
            return "unknown status";
    }
}

const char* nanoep_last_hip_error(void) {
    return g_last_hip_error == hipSuccess ? "" : hipGetErrorString(g_last_hip_error);
}

int nanoep_set_tuning(const char* name, int value) {
    const int at = find_switch(name);
    if (at < 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    std::call_once(g_switches_once, load_switches_from_environment);
    g_switch_values[at].store(value, std::memory_order_relaxed);
    return NANOEP_OK;
}

int nanoep_get_tuning(const char* name, int* value) {
    const int at = find_switch(name);
    if (at < 0 || value == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    std::call_once(g_switches_once, load_switches_from_environment);
    *value = g_switch_values[at].load(std::memory_order_relaxed);
    return NANOEP_OK;
}

void nanoep_reset_tuning(void) {
    std::call_once(g_switches_once, load_switches_from_environment);
    load_switches_from_environment();
}

int nanoep_device_topology(int* out_cus, int* out_xcds, int64_t* out_l2_bytes) {
    const Topology topology = current_topology(current_tuning());
    if (out_cus != nullptr)
        *out_cus = topology.cus;
    if (out_xcds != nullptr)
        *out_xcds = topology.xcds;
    if (out_l2_bytes != nullptr)
        *out_l2_bytes = topology.l2_bytes;
    return NANOEP_OK;
}

int nanoep_device_cu_count(int device, int* out_cus) {
    if (out_cus == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    NANOEP_HIP_TRY(hipDeviceGetAttribute(out_cus, hipDeviceAttributeMultiprocessorCount, device));
    return NANOEP_OK;
}

int nanoep_window_layout(int ranks, int64_t max_tokens, int hidden, int topk, int64_t num_experts,
                         int allow_multiple_reduction, int64_t out[5]) {
    if (out == nullptr || ranks <= 0 || ranks > 32 || max_tokens <= 0 || hidden <= 0 || topk <= 0 || topk > 32)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (num_experts <= 0 || num_experts % ranks != 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    // 32-byte fields: per-rank barrier signals, packed notify reductions, int64 counts
    // (rank counts, per-source expert counts, send cursors), then one arena shared by the
    // dispatch wire rows and the combine return rows.
    const auto up32 = [](int64_t v) { return (v + 31) / 32 * 32; };
    const int64_t notify_bytes = (static_cast<int64_t>(ranks) + num_experts) * 8;
    const int64_t reduction_offset = up32(static_cast<int64_t>(ranks) * 8);
    const int64_t count_offset = up32(reduction_offset + notify_bytes);
    const int64_t payload_offset = up32(count_offset + notify_bytes + static_cast<int64_t>(ranks) * 8);
    const int64_t wire_weights = up32(32 + static_cast<int64_t>(topk) * 8);
    const int64_t wire_x = up32(wire_weights + static_cast<int64_t>(topk) * 4);
    const int64_t wire_row = up32(wire_x + static_cast<int64_t>(hidden) * 2);
    const int64_t return_row = up32(up32(static_cast<int64_t>(hidden) * 2) + static_cast<int64_t>(topk) * 4);
    const int64_t partitions = allow_multiple_reduction ? (ranks < topk ? ranks : topk) : topk;
    const int64_t wire_bytes = static_cast<int64_t>(ranks) * max_tokens * wire_row;
    const int64_t return_bytes = partitions * max_tokens * return_row;
    out[0] = 0;
    out[1] = count_offset;
    out[2] = payload_offset;
    out[3] = payload_offset;
    out[4] = up32(payload_offset + (wire_bytes > return_bytes ? wire_bytes : return_bytes));
    return NANOEP_OK;
}

int nanoep_copy_bytes(const void* src, void* dst, size_t bytes, void* stream_handle) {
    if (bytes % 16 != 0 || !aligned16(src) || !aligned16(dst))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (bytes == 0)
        return NANOEP_OK;
    if (src == nullptr || dst == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const size_t vectors = bytes / 16;
    const size_t blocks = (vectors + kBlockThreads - 1) / kBlockThreads;
    if (blocks > UINT32_MAX)
        return NANOEP_ERR_INVALID_ARGUMENT;
    copy_vectors_kernel<<<static_cast<unsigned>(blocks), kBlockThreads, 0, static_cast<hipStream_t>(stream_handle)>>>(
        static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), vectors);
    NANOEP_HIP_TRY(hipGetLastError());
    return NANOEP_OK;
}

}  // extern "C"
