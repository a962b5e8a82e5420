// Version, status strings, window layout, profiler calibration copy.

#include <unistd.h>

#include "nanoep_device.h"

extern char** environ;

namespace nanoep {

thread_local hipError_t g_last_hip_error = hipSuccess;
thread_local Tuning g_tuning;

void refresh_tuning() {
    Tuning fresh;
    struct Switch {
        const char* name;  // behind the NANOEP_ prefix
        int* value;
    };
    const Switch switches[] = {
        {"CHUNKS_PER_BLOCK", &fresh.chunks_per_block}, {"ROWS_PER_BLOCK", &fresh.rows_per_block},
        {"DISPATCH_ORDER", &fresh.dispatch_order},     {"DISPATCH_SPAN", &fresh.dispatch_span},
        {"DISPATCH_SIDE", &fresh.dispatch_side},       {"DISPATCH_WHOLE_ROWS", &fresh.dispatch_whole_rows},
        {"LAYOUT_LAUNCHES", &fresh.layout_launches},   {"WINDOW_TOKENS", &fresh.window_tokens},
    };
    if (environ != nullptr) {
        for (char** entry = environ; *entry != nullptr; ++entry) {
            const char* text = *entry;
            if (text[0] != 'N' || std::strncmp(text, "NANOEP_", 7) != 0)
                continue;
            for (const Switch& item : switches) {
                const size_t length = std::strlen(item.name);
                // NANOEP_<NAME>=<number>; an empty value leaves the default
                if (std::strncmp(text + 7, item.name, length) == 0 && text[7 + length] == '=' && text[8 + length] != '\0')
                    *item.value = std::atoi(text + 8 + length);
            }
        }
    }
    g_tuning = fresh;
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
