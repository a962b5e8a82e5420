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
    {"LAYOUT_LAUNCHES", &Tuning::layout_launches},   {"WINDOW_TOKENS", &Tuning::window_tokens},
    {"RECALL_ORDER", &Tuning::recall_order},         {"FRESH_OUTPUTS", &Tuning::fresh_outputs},
    {"REBUILD_ORDER", &Tuning::rebuild_order},       {"XCDS", &Tuning::xcds},
    {"L2_BYTES", &Tuning::l2_bytes},                 {"DISPATCH_PREFETCH", &Tuning::dispatch_prefetch},
    {"COMBINE_STORES", &Tuning::combine_stores},     {"DISPATCH_PACK", &Tuning::dispatch_pack}, {"COMBINE_UNITS", &Tuning::combine_units},
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
            held_combine_residency(asked.held_wavefronts);
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

// Plain streams in the shape of the row kernels: one wavefront per 1 KiB chunk of a destination row,
// workgroups of a chosen number of consecutive chunks (a whole row, a part of one, or several short
// rows), one 128-bit access per lane, nontemporal stores, workgroups dealt to the XCDs in contiguous
// ranges.  They move the bytes of a dispatch or a combine with addresses that are a
// closed form of the workgroup index and no lookups: what such a launch attains is the ceiling a
// permute of the same bytes can approach.
//   kStreamRead   : reads src row r (nothing is written unless a lane holds an impossible value)
//   kStreamFill   : writes dst row r
//   kStreamFanOut : every source row is written kFan times.  Rows go in windows of `window` source
//                   rows: destination row r = w * window * kFan + p * window + i holds source row
//                   w * window + i (kFan passes over a window that can stay in an XCD's L2, as the
//                   slot-order walk makes them; window == 1: kFan neighbours share a row).
//   kStreamFanIn  : destination row w * window + i is the integer sum of the kFan source rows
//                   w * window * kFan + p * window + i (kFan linear streams per window).
enum StreamKind { kStreamRead = 0, kStreamFill = 1, kStreamFanOut = 2, kStreamFanIn = 3 };

template <int kKind, int kFan>
__global__ void __launch_bounds__(1024) stream_probe_kernel(const u32x4* __restrict__ src,
                                                            u32x4* __restrict__ dst,
                                                            uint32_t dst_rows,
                                                            uint32_t row_vectors,
                                                            uint32_t window,
                                                            uint32_t span_magic,  // fast divisor by window * kFan
                                                            uint32_t span_shift,
                                                            uint32_t window_magic,  // fast divisor by window
                                                            uint32_t window_shift,
                                                            uint32_t blocks_per_xcd,
                                                            uint32_t chunks,  // 1 KiB chunks of a row
                                                            uint32_t chunks_magic,
                                                            uint32_t chunks_shift,
                                                            XcdMap xcds) {
    NANOEP_FETCH_ARGS_4(src, dst, dst_rows, row_vectors);
    NANOEP_FETCH_ARGS_4(window, span_magic, span_shift, blocks_per_xcd);
    NANOEP_FETCH_ARGS_4(xcds.count, xcds.magic, xcds.shift, window_magic);
    NANOEP_FETCH_ARGS_4(chunks, chunks_magic, chunks_shift, window_shift);
    const uint32_t index_in_xcd = fast_divide(blockIdx.x, xcds.magic, xcds.shift);
    const uint32_t xcd = blockIdx.x - index_in_xcd * xcds.count;
    if (index_in_xcd >= blocks_per_xcd)
        return;
    const uint32_t unit = (xcd * blocks_per_xcd + index_in_xcd) * blockDim.y + __builtin_amdgcn_readfirstlane(threadIdx.y);
    const uint32_t row = fast_divide(unit, chunks_magic, chunks_shift);
    if (row >= dst_rows)
        return;
    const uint32_t vector = (unit - row * chunks) * kWave + threadIdx.x;
    const bool in_row = vector < row_vectors;
    const uint32_t at = in_row ? vector : 0u;
    u32x4* out = dst + static_cast<uint64_t>(row) * row_vectors + vector;
    if (kKind == kStreamRead) {
        const u32x4 data = load_vec<true>(src + static_cast<uint64_t>(row) * row_vectors + at);
        if (data.x == 0x7fc1a5a5u && data.y == 0x12345678u && data.z == 0x9abcdef0u && in_row)
            store_vec<true>(out, data);
    } else if (kKind == kStreamFill) {
        const u32x4 data = {row, vector, 0u, 0u};
        if (in_row)
            store_vec<true>(out, data);
    } else if (kKind == kStreamFanOut) {
        const uint32_t in_window = fast_divide(row, span_magic, span_shift);
        const uint32_t rest = row - in_window * window * kFan;
        const uint32_t from = in_window * window + (rest - fast_divide(rest, window_magic, window_shift) * window);
        const u32x4 data = src[static_cast<uint64_t>(from) * row_vectors + at];
        if (in_row)
            store_vec<true>(out, data);
    } else {
        const uint32_t in_window = fast_divide(row, window_magic, window_shift);
        const uint64_t first = static_cast<uint64_t>(in_window) * window * kFan + (row - in_window * window);
        u32x4 data[kFan];
#pragma unroll
        for (int p = 0; p < kFan; ++p)
            data[p] = load_vec<true>(src + (first + static_cast<uint64_t>(p) * window) * row_vectors + at);
        u32x4 sum = data[0];
#pragma unroll
        for (int p = 1; p < kFan; ++p)
            sum += data[p];
        if (in_row)
            store_vec<true>(out, sum);
    }
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

int nanoep_stream_probe(int kind, const void* src, void* dst, int64_t dst_rows, int hidden, int fan, int64_t window,
                        int waves_per_block, void* stream_handle) {
    if (kind < kStreamRead || kind > kStreamFanIn || hidden <= 0 || hidden % 8 != 0 || hidden > 8192 || dst_rows <= 0 ||
        dst_rows >= (int64_t{1} << 31) - 64 || window < 1 || window * fan >= (int64_t{1} << 31) || !aligned16(src) || !aligned16(dst))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if ((fan != 1 && fan != 2 && fan != 4 && fan != 7 && fan != 8) || waves_per_block < 0 || waves_per_block > kMaxWavesPerBlock)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if ((kind != kStreamFill && src == nullptr) || dst == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    // whole windows only: every destination row then has all its source rows
    if (kind == kStreamFanOut ? dst_rows % (window * fan) != 0 : kind == kStreamFanIn && dst_rows % window != 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const Topology topology = current_topology(current_tuning());
    const XcdMap xcds = make_xcd_map(topology.xcds);
    const uint32_t row_vectors = static_cast<uint32_t>(hidden / 8);
    const uint32_t chunks = (row_vectors + kWave - 1) / kWave;
    // 0: a workgroup per row (rows of up to 16 chunks), else that many consecutive chunks a workgroup
    const uint32_t waves = waves_per_block > 0 ? static_cast<uint32_t>(waves_per_block) : (chunks < kMaxWavesPerBlock ? chunks : kMaxWavesPerBlock);
    const int64_t blocks = (dst_rows * chunks + waves - 1) / waves;
    if (blocks >= (int64_t{1} << 31) - 64 || dst_rows * chunks >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const uint32_t per_xcd = static_cast<uint32_t>((blocks + xcds.count - 1) / xcds.count);
    const FastDivisor span_divisor = make_fast_divisor(static_cast<uint32_t>(window * fan));
    const FastDivisor window_divisor = make_fast_divisor(static_cast<uint32_t>(window));
    const FastDivisor chunks_divisor = make_fast_divisor(chunks);
    const dim3 grid(per_xcd * xcds.count), block(kWave, waves, 1);
    auto stream = static_cast<hipStream_t>(stream_handle);
#define NANOEP_LAUNCH_STREAM(KIND, FAN)                                                                                  \
    stream_probe_kernel<KIND, FAN><<<grid, block, 0, stream>>>(                                                          \
        static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), static_cast<uint32_t>(dst_rows), row_vectors,          \
        static_cast<uint32_t>(window), span_divisor.magic, span_divisor.shift, window_divisor.magic, window_divisor.shift, \
        per_xcd, chunks, chunks_divisor.magic, chunks_divisor.shift, xcds)
#define NANOEP_LAUNCH_STREAM_FAN(KIND)         \
    switch (fan) {                             \
        case 1:                                \
            NANOEP_LAUNCH_STREAM(KIND, 1);     \
            break;                             \
        case 2:                                \
            NANOEP_LAUNCH_STREAM(KIND, 2);     \
            break;                             \
        case 4:                                \
            NANOEP_LAUNCH_STREAM(KIND, 4);     \
            break;                             \
        case 7:                                \
            NANOEP_LAUNCH_STREAM(KIND, 7);     \
            break;                             \
        default:                               \
            NANOEP_LAUNCH_STREAM(KIND, 8);     \
            break;                             \
    }
    if (kind == kStreamRead)
        NANOEP_LAUNCH_STREAM(kStreamRead, 1);
    else if (kind == kStreamFill)
        NANOEP_LAUNCH_STREAM(kStreamFill, 1);
    else if (kind == kStreamFanOut)
        NANOEP_LAUNCH_STREAM_FAN(kStreamFanOut)
    else
        NANOEP_LAUNCH_STREAM_FAN(kStreamFanIn)
#undef NANOEP_LAUNCH_STREAM_FAN
#undef NANOEP_LAUNCH_STREAM
    NANOEP_HIP_TRY(hipGetLastError());
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
