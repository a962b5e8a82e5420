// Routing layout: per-expert histograms, device-wide scan, stable token-order slots, slot-order list.

#include <ctime>

#include <mutex>

#include "nanoep_device.h"

// Device memory of nanoep_layout_static: the layout kernels' workspace (block histograms, in-block
// ranks, receive rows) for callers that cannot allocate.  Every GPU holds its own copy of the array
// at its own address until the process ends; host code only ever uses the address that
// hipGetSymbolAddress returns for the current device, never the array's name.
static __device__ __align__(256) unsigned char scratch[NANOEP_STATIC_SCRATCH_BYTES];

namespace nanoep {
namespace {

// Largest block of tokens a layout workgroup handles (one thread per token).
constexpr int kMaxBlockTokens = 256;
// What the launch plans below depend on besides the batch: the forced settings and the device's XCD
// count and L2 size (the rows of one window should fit an XCD's L2, since the dispatch walks the
// slot-order list window by window and wants every re-use of a source row to hit that cache).
struct Knobs {
    int window_tokens;
    int layout_launches;
    int xcds;
    int64_t l2_bytes;
};

Knobs current_knobs() {
    const Tuning tuning = current_tuning();
    const Topology topology = current_topology(tuning);
    return {tuning.window_tokens, tuning.layout_launches, topology.xcds, topology.l2_bytes};
}

// Most blocks for which every assignment workgroup scans the block histograms itself.
constexpr int kFusedScanMaxBlocks = 1024;
// Largest window: the run of consecutive tokens the slot-order list is ordered by.
constexpr int kMaxWindowTokens = 1024;

// Tokens of one window of the slot-order list.
//  * `hidden` (bf16 elements of a payload row, 0 = not known) sizes the window so that its rows fit an
//    XCD's L2 with a sixteenth to spare for the write stream (a window that fills the L2 to the
//    brim loses what the prefetch brought in: 4096 x 4096 top-2 18.9 -> 18.3 us cold, 14.9 -> 12.8 us
//    cache resident with half the window): 512 tokens up to 3840 elements, 256 up to 7680 (and when
//    it is not known), then 128, 64.
//    Rows of up to 1024 elements take 1024 tokens (half the L2: at 2048 elements a 1024-token window
//    measured 8 % slower than a 512-token one, at 1024 and 512 elements 5 and 7 % faster).
//  * The dispatch hands every XCD whole windows when there are at least as many as XCDs (twice as
//    many for 1024-token windows): batches of more than 256 tokens take smaller windows (down to 64
//    tokens) to get there.
// (sizes above are those of a 4 MiB L2 and 8 XCDs)
int layout_window_tokens(int64_t tokens_total, int hidden, const Knobs& knobs) {
    // WINDOW_TOKENS forces a window: any multiple of 32 up to 256 (one layout workgroup), or 512 / 1024
    const int forced = knobs.window_tokens;
    if (forced >= 32 && forced % 32 == 0 && (forced <= 256 || forced == 512 || forced == 1024) && tokens_total > 256)
        return forced;
    int window = 256;
    if (hidden > 0)
        for (window = kMaxWindowTokens;
             window > 64 && static_cast<int64_t>(window) * hidden * 2 > (window > 512 ? knobs.l2_bytes / 2 : knobs.l2_bytes - knobs.l2_bytes / 16);
             window /= 2) {
        }
    if (tokens_total <= 256 && window > 256)
        window = 256;  // one layout block: the whole layout is then a single launch
    while (tokens_total > 256 && window > 64 && (tokens_total + window - 1) / window < (window > 512 ? 2 * knobs.xcds : knobs.xcds))
        window /= 2;
    return window;
}

// Tokens handled by one layout workgroup (one thread per token): the window, at most 256, fewer when
// the LDS bit matrix ((L+1) rows of tokens/32 words plus a 16-bit prefix per word) asks for it.  A
// window of 512 tokens is two workgroups' worth: the assignment pass orders the list by windows from
// the block histograms (a 512-token workgroup makes the dispatch as fast and the layout 5 us slower).
int layout_tokens_per_block(int64_t tokens_total, int64_t local_experts, int hidden, const Knobs& knobs) {
    if (static_cast<size_t>(local_experts + 1) * 16 > kLayoutLdsBudget)  // four int32 arrays of the assignment kernel
        return 0;
    const int window = layout_window_tokens(tokens_total, hidden, knobs);
    for (int tokens = window < kMaxBlockTokens ? window : kMaxBlockTokens; tokens >= 32; tokens = tokens / 2 / 32 * 32) {
        const size_t words = static_cast<size_t>(tokens / 32);
        if (static_cast<size_t>(local_experts + 1) * (words * 6 + 4) <= kLayoutLdsBudget)
            return tokens;
    }
    return 0;
}

// Layout blocks per window.  Windows of several blocks need every assignment workgroup to see the
// block histograms (the two-launch plan); with a separate scan launch the window is the block.
int layout_window_blocks(int64_t tokens_total, int64_t local_experts, int hidden, bool fused_scan, const Knobs& knobs) {
    const int per_block = layout_tokens_per_block(tokens_total, local_experts, hidden, knobs);
    const int window = layout_window_tokens(tokens_total, hidden, knobs);
    return per_block == 0 || !fused_scan || window <= per_block ? 1 : window / per_block;
}

// Whether the layout of this batch runs as two launches (see nanoep_layout).
bool layout_uses_fused_scan(int64_t tokens_total, int64_t local_experts, int hidden, const Knobs& knobs) {
    const int per_block = layout_tokens_per_block(tokens_total, local_experts, hidden, knobs);
    if (per_block == 0 || tokens_total == 0)
        return false;
    const int64_t blocks = (tokens_total + per_block - 1) / per_block;
    const int forced = knobs.layout_launches;
    if (forced == 3)
        return false;
    return forced == 2 || blocks <= kFusedScanMaxBlocks;
}

// Smallest block any `hidden` can lead to for this batch: what the workspace is sized for.
int layout_smallest_block(int64_t tokens_total, int64_t local_experts, const Knobs& knobs) {
    const int narrow = layout_tokens_per_block(tokens_total, local_experts, 1 << 20, knobs);
    const int wide = layout_tokens_per_block(tokens_total, local_experts, 8, knobs);
    return narrow < wide ? narrow : wide;
}

struct LayoutWorkspace {
    int32_t* block_counts;  // [NB][L+1]; column L counts tokens with any valid choice
    int32_t* block_status;  // [NB]
    int32_t* packed_rank;   // [T][K]  (expert << 8) | in-block rank, or -1
    int32_t* local_row;     // [T]
    int64_t* totals;        // [1] total assignments, handed from the scan kernel to the assignment kernel
    size_t bytes;
};

LayoutWorkspace carve_layout_workspace(void* base, int64_t tokens, int topk, int64_t local_experts, const Knobs& knobs) {
    const int per_block = layout_smallest_block(tokens, local_experts, knobs);
    const int64_t blocks = per_block == 0 ? 0 : (tokens + per_block - 1) / per_block;
    auto* cursor = static_cast<uint8_t*>(base);
    size_t offset = 0;
    LayoutWorkspace ws{};
    ws.block_counts = reinterpret_cast<int32_t*>(cursor + offset);
    offset = align_up(offset + static_cast<size_t>(blocks) * (local_experts + 1) * 4, 256);
    ws.block_status = reinterpret_cast<int32_t*>(cursor + offset);
    offset = align_up(offset + static_cast<size_t>(blocks) * 4, 256);
    ws.packed_rank = reinterpret_cast<int32_t*>(cursor + offset);
    offset = align_up(offset + static_cast<size_t>(tokens) * topk * 4, 256);
    ws.local_row = reinterpret_cast<int32_t*>(cursor + offset);
    offset = align_up(offset + static_cast<size_t>(tokens) * 4, 256);
    ws.totals = reinterpret_cast<int64_t*>(cursor + offset);
    offset = align_up(offset + 8, 256);
    ws.bytes = offset + 256;
    return ws;
}

// A (token, k) entry of the rank table packs (expert << kRankBits) | in-block rank; -1 marks a
// masked choice.  A layout block never holds more than 256 tokens, so the rank fits 8 bits.
constexpr int kRankBits = 8;
static_assert(kMaxBlockTokens <= (1 << kRankBits), "in-block ranks must fit the packed entry");
constexpr int kRankMask = (1 << kRankBits) - 1;

// One thread per token.  bits[e][w] has bit (token & 31) of word (token >> 5) set when the token
// chose expert e; row L marks tokens with any valid choice.  Experts inside a token are distinct,
// so the order of one expert's assignments is the token order and a popcount prefix is the rank.
// The token's routing ids are fetched in one batch of independent loads (kCap >= K of them, the
// surplus re-reads id 0) and stay in registers for both passes over the bit matrix.
// What a thread of the count pass knows at its end, for a kernel that goes on to the assignment
// pass in the same workgroup and need not read it back from memory.
template <int kCap>
struct CountedToken {
    int32_t packed[kCap];  // the token's entries of the rank table
    int32_t row;           // the token's receive row within the block, -1 when it is not sent
    int32_t first_count;   // the block's count of histogram row threadIdx.x (0 when there is no such row)
    int32_t bad;           // the block's routing status bits
};

template <int kCap>
__device__ __forceinline__ void layout_count_block(const int64_t* __restrict__ topk_idx,
                                                   int64_t num_tokens,
                                                   int num_topk,
                                                   int local_experts,
                                                   int words,
                                                   int threads,
                                                   int64_t* __restrict__ snapshot,
                                                   int32_t* block_counts,
                                                   int32_t* block_status,
                                                   int32_t* packed_rank,
                                                   int32_t* local_row,
                                                   CountedToken<kCap>& counted) {
    extern __shared__ uint32_t layout_lds[];
    const int rows = local_experts + 1;
    // bit rows are words + 1 apart: an odd stride spreads the experts a wavefront touches over the LDS banks
    const int stride = words + 1;
    uint32_t* bits = layout_lds;
    auto* prefix = reinterpret_cast<uint16_t*>(bits + static_cast<size_t>(rows) * stride);
    __shared__ int block_bad;

    const int tokens_per_block = words * 32;
    const int local_token = threadIdx.x;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * tokens_per_block + local_token;
    const bool live = local_token < tokens_per_block && token < num_tokens;
    const int word = local_token >> 5;
    const uint32_t bit = 1u << (local_token & 31);

    typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
    typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
    // rows of an even number of ids start 16-byte aligned when the tensor does: two ids a load and a store
    const bool wide_ids = (num_topk & 1) == 0 && (reinterpret_cast<uintptr_t>(topk_idx) & 15) == 0;
    const bool wide_snapshot = (num_topk & 1) == 0 && (reinterpret_cast<uintptr_t>(snapshot) & 15) == 0;
    int64_t raw[kCap];
    const int64_t* mine = topk_idx + (live ? token : 0) * num_topk;
    if (wide_ids) {
#pragma unroll
        for (int k = 0; k < kCap; k += 2) {
            const i64x2 pair = *reinterpret_cast<const i64x2*>(mine + (k < num_topk ? k : 0));
            raw[k] = pair.x;
            raw[k + 1] = pair.y;
        }
    } else {
#pragma unroll
        for (int k = 0; k < kCap; ++k)
            raw[k] = mine[k < num_topk ? k : 0];
    }

    for (int i = threadIdx.x; i < rows * stride; i += threads)
        bits[i] = 0;
    if (threadIdx.x == 0)
        block_bad = 0;
    __syncthreads();

    int ids[kCap];  // expert id, -1 masked, -2 out of range
#pragma unroll
    for (int k = 0; k < kCap; ++k) {
        const int64_t expert = raw[k];
        ids[k] = (expert >= 0 && expert < local_experts) ? static_cast<int>(expert) : (expert == -1 ? -1 : -2);
        if (!live || k >= num_topk)
            ids[k] = -1;
        else if (!wide_snapshot)
            snapshot[token * num_topk + k] = expert;
    }
    if (live && wide_snapshot) {
#pragma unroll
        for (int k = 0; k < kCap; k += 2)
            if (k < num_topk)
                *reinterpret_cast<i64x2*>(snapshot + token * num_topk + k) = i64x2{raw[k], raw[k + 1]};
    }

    int bad = 0;
    bool any = false;
#pragma unroll
    for (int k = 0; k < kCap; ++k) {
        const int id = ids[k];
        if (id >= 0) {
            const uint32_t old = atomicOr(&bits[static_cast<size_t>(id) * stride + word], bit);
            if (old & bit)
                bad |= NANOEP_ROUTING_DUPLICATE;
            any = true;
        } else if (id == -2) {
            bad |= NANOEP_ROUTING_BAD_EXPERT;
        }
    }
    if (any)
        atomicOr(&bits[static_cast<size_t>(local_experts) * stride + word], bit);
    if (bad)
        atomicOr(&block_bad, bad);
    __syncthreads();

    counted.first_count = 0;
    for (int row = threadIdx.x; row < rows; row += threads) {
        int running = 0;
        for (int w = 0; w < words; ++w) {
            prefix[static_cast<size_t>(row) * words + w] = static_cast<uint16_t>(running);
            running += __popc(bits[static_cast<size_t>(row) * stride + w]);
        }
        block_counts[static_cast<int64_t>(blockIdx.x) * rows + row] = running;
        if (row == static_cast<int>(threadIdx.x))
            counted.first_count = running;
    }
    if (threadIdx.x == 0)
        block_status[blockIdx.x] = block_bad;
    __syncthreads();
    counted.bad = block_bad;
    counted.row = -1;
#pragma unroll
    for (int k = 0; k < kCap; ++k)
        counted.packed[k] = -1;

    if (live) {
        const uint32_t below = bit - 1;
        int32_t packed[kCap];
#pragma unroll
        for (int k = 0; k < kCap; ++k) {
            const int id = ids[k];
            packed[k] = -1;
            if (id >= 0) {
                const int rank = prefix[static_cast<size_t>(id) * words + word] +
                                 __popc(bits[static_cast<size_t>(id) * stride + word] & below);
                packed[k] = (id << kRankBits) | rank;
            }
        }
        if ((num_topk & 3) == 0 && (reinterpret_cast<uintptr_t>(packed_rank) & 15) == 0) {
#pragma unroll
            for (int k = 0; k < kCap; k += 4)
                if (k < num_topk)
                    *reinterpret_cast<i32x4*>(packed_rank + token * num_topk + k) = i32x4{packed[k], packed[k + 1], packed[k + 2], packed[k + 3]};
        } else {
#pragma unroll
            for (int k = 0; k < kCap; ++k)
                if (k < num_topk)
                    packed_rank[token * num_topk + k] = packed[k];
        }
        const uint32_t received = bits[static_cast<size_t>(local_experts) * stride + word];
        counted.row = (received & bit) ? prefix[static_cast<size_t>(local_experts) * words + word] + __popc(received & below) : -1;
        local_row[token] = counted.row;
#pragma unroll
        for (int k = 0; k < kCap; ++k)
            counted.packed[k] = packed[k];
    }
}

template <int kCap>
__global__ void __launch_bounds__(kMaxBlockTokens) layout_count_kernel(const int64_t* __restrict__ topk_idx,
                                                           int64_t num_tokens,
                                                           int num_topk,
                                                           int local_experts,
                                                           int words,
                                                           int threads,
                                                           int64_t* __restrict__ snapshot,
                                                           int32_t* __restrict__ block_counts,
                                                           int32_t* __restrict__ block_status,
                                                           int32_t* __restrict__ packed_rank,
                                                           int32_t* __restrict__ local_row) {
    CountedToken<kCap> counted;
    layout_count_block<kCap>(topk_idx, num_tokens, num_topk, local_experts, words, threads, snapshot, block_counts,
                             block_status, packed_rank, local_row, counted);
}

__device__ __forceinline__ int64_t round_up_to(int64_t value, int64_t alignment) {
    return alignment == 1 ? value : (value + alignment - 1) / alignment * alignment;
}

// Single workgroup.  Phase 1 turns every column of block_counts into its exclusive prefix over
// blocks (threads are spread over columns x block segments so small expert counts still use the
// whole workgroup).  Phase 2 scans the aligned expert totals.  The mailbox word 0 is stored last.
__global__ void __launch_bounds__(kScanThreads) layout_scan_kernel(int32_t* __restrict__ block_counts,
                                                                  const int32_t* __restrict__ block_status,
                                                                  int num_blocks,
                                                                  int local_experts,
                                                                  int64_t alignment,
                                                                  int64_t* __restrict__ expert_counts,
                                                                  int64_t* __restrict__ expert_offsets,
                                                                  int64_t* __restrict__ send_counts,
                                                                  int64_t* __restrict__ recv_rank_prefix,
                                                                  int64_t* __restrict__ totals,
                                                                  int64_t* host_counts) {
    extern __shared__ int32_t column_total[];  // [L+1]
    __shared__ int32_t partial[kScanThreads];
    __shared__ int64_t scan[kScanThreads];
    __shared__ int64_t assignments[kScanThreads];
    __shared__ int status_bits;

    const int tid = threadIdx.x;
    const int rows = local_experts + 1;
    if (tid == 0)
        status_bits = 0;

    const int columns_per_pass = rows < kScanThreads ? rows : kScanThreads;
    const int segments = kScanThreads / columns_per_pass;
    const int blocks_per_segment = (num_blocks + segments - 1) / segments;
    for (int column0 = 0; column0 < rows; column0 += columns_per_pass) {
        const int column_local = tid % columns_per_pass;
        const int segment = tid / columns_per_pass;
        const int column = column0 + column_local;
        const bool active = segment < segments && column < rows;
        const int begin = segment * blocks_per_segment;
        const int end = begin + blocks_per_segment < num_blocks ? begin + blocks_per_segment : num_blocks;
        int sum = 0;
        if (active)
            for (int b = begin; b < end; ++b)
                sum += block_counts[static_cast<int64_t>(b) * rows + column];
        partial[tid] = active ? sum : 0;
        __syncthreads();
        if (active) {
            int running = 0;
            for (int s = 0; s < segment; ++s)
                running += partial[s * columns_per_pass + column_local];
            for (int b = begin; b < end; ++b) {
                const int64_t at = static_cast<int64_t>(b) * rows + column;
                const int count = block_counts[at];
                block_counts[at] = running;
                running += count;
            }
            if (segment == segments - 1)
                column_total[column] = running;
        }
        __syncthreads();
    }

    int bad = 0;
    for (int b = tid; b < num_blocks; b += kScanThreads)
        bad |= block_status[b];
    if (bad)
        atomicOr(&status_bits, bad);

    const int per_thread = (local_experts + kScanThreads - 1) / kScanThreads;
    const int first = tid * per_thread;
    const int last = first + per_thread < local_experts ? first + per_thread : local_experts;
    int64_t padded_sum = 0, count_sum = 0;
    for (int e = first; e < last; ++e) {
        const int64_t count = column_total[e];
        count_sum += count;
        padded_sum += round_up_to(count, alignment);
    }
    scan[tid] = padded_sum;
    assignments[tid] = count_sum;
    __syncthreads();
    for (int step = 1; step < kScanThreads; step *= 2) {
        const int64_t add_scan = tid >= step ? scan[tid - step] : 0;
        const int64_t add_assign = tid >= step ? assignments[tid - step] : 0;
        __syncthreads();
        scan[tid] += add_scan;
        assignments[tid] += add_assign;
        __syncthreads();
    }
    int64_t running = scan[tid] - padded_sum;
    for (int e = first; e < last; ++e) {
        const int64_t count = column_total[e];
        expert_counts[e] = count;
        expert_offsets[e] = running;
        running += round_up_to(count, alignment);
    }
    if (tid == 0) {
        const int64_t received = column_total[local_experts];
        const int64_t capacity = scan[kScanThreads - 1];
        expert_offsets[local_experts] = capacity;
        send_counts[0] = received;
        recv_rank_prefix[0] = received;
        totals[0] = assignments[kScanThreads - 1];
        host_counts[1] = capacity;
        host_counts[2] = assignments[kScanThreads - 1];
        host_counts[3] = status_bits;
        __threadfence_system();
        __hip_atomic_store(&host_counts[0], received, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// Writes one token's part of the handle.  `packed` holds the token's entries of the rank table,
// `slot_base[e]` is the first slot of this block's
// assignments to expert e; `order_base[e]` is where expert e's run starts in the block's segment
// of the slot-order list (`order` points at that segment, or is null).
template <int kCap>
__device__ __forceinline__ void assign_token_slots(int64_t token,
                                                   int num_topk,
                                                   int expand,
                                                   int row_in_block,
                                                   int64_t row_base,
                                                   const int32_t* slot_base,
                                                   const int32_t* order_base,
                                                   const int32_t (&packed)[kCap],
                                                   int32_t* __restrict__ recv_metadata,
                                                   int64_t* __restrict__ dst_slots,
                                                   int32_t* __restrict__ token_slots,
                                                   int64_t* __restrict__ order) {
    typedef int32_t i32x2 __attribute__((ext_vector_type(2)));
    typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
    // a token's row of the slot table: wide stores where the row width keeps them aligned
    const auto store_table_row = [&](const int32_t (&values)[kCap]) {
        if (token_slots == nullptr)
            return;
        int32_t* row = token_slots + token * num_topk;
        if ((num_topk & 3) == 0 && (reinterpret_cast<uintptr_t>(token_slots) & 15) == 0) {
#pragma unroll
            for (int k = 0; k < kCap; k += 4)
                if (k < num_topk)
                    *reinterpret_cast<i32x4*>(row + k) = i32x4{values[k], values[k + 1], values[k + 2], values[k + 3]};
        } else {
#pragma unroll
            for (int k = 0; k < kCap; ++k)
                if (k < num_topk)
                    row[k] = values[k];
        }
    };
    int32_t values[kCap];
#pragma unroll
    for (int k = 0; k < kCap; ++k)
        values[k] = -1;
    if (row_in_block < 0) {
        dst_slots[token] = -1;
        store_table_row(values);
        return;
    }
    const int64_t row = row_base + row_in_block;
    dst_slots[token] = row;
#pragma unroll
    for (int k = 0; k < kCap; ++k) {
        if (k >= num_topk)
            break;
        if (packed[k] >= 0) {
            const int expert = packed[k] >> kRankBits;
            const int rank = packed[k] & kRankMask;
            values[k] = expand ? slot_base[expert] + rank : expert;
            if (order != nullptr) {
                const uint32_t source = static_cast<uint32_t>(token * num_topk + k);
                order[order_base[expert] + rank] = (static_cast<int64_t>(values[k]) << 32) | source;
            }
        }
    }
    // the receive row [0, token, K values]: pairs of words when K is even and the table 8-byte aligned (every row then is)
    int32_t* out = recv_metadata + row * (num_topk + 2);
    if ((num_topk & 1) == 0 && (reinterpret_cast<uintptr_t>(recv_metadata) & 7) == 0) {
        *reinterpret_cast<i32x2*>(out) = i32x2{0, static_cast<int32_t>(token)};
#pragma unroll
        for (int k = 0; k < kCap; k += 2)
            if (k < num_topk)
                *reinterpret_cast<i32x2*>(out + 2 + k) = i32x2{values[k], values[k + 1]};
    } else {
        out[0] = 0;
        out[1] = static_cast<int32_t>(token);
#pragma unroll
        for (int k = 0; k < kCap; ++k)
            if (k < num_topk)
                out[2 + k] = values[k];
    }
    store_table_row(values);
}

__device__ __forceinline__ int64_t wave_inclusive_scan(int64_t value) {
    const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
    for (int distance = 1; distance < kWave; distance *= 2) {
        const int64_t other = __shfl_up(value, distance, kWave);
        if (lane >= distance)
            value += other;
    }
    return value;
}

// Slot assignment, one workgroup per block of tokens (the blocks of layout_count_kernel).
//
// kFusedScan: `block_counts` holds the raw block histograms and every workgroup sums them itself
// (they sit in L2): per column the total over all blocks and the part from the blocks before its
// own, then the aligned exclusive scan over experts, all in LDS; the workgroup whose index is
// `publisher` also writes the per-expert outputs and the host mailbox (word 0 last).  With several
// blocks that is one more workgroup behind those of the blocks, which has no tokens of its own: the
// store to host memory and its fence then sit on nobody's way to the token writes.  Otherwise
// layout_scan_kernel has done that and `block_counts` holds each block's exclusive prefixes.
//
// Either way the workgroup also scans its own histogram over experts: that places every
// assignment of the block in expert-major order inside the block's run of `slot_order`; the runs
// of consecutive blocks follow each other without gaps and the unused tail of the list is -1.
template <int kCap, bool kFusedScan, bool kOwnBlock = false>
__device__ __forceinline__ void layout_assign_block(const int32_t* block_counts,
                                                    const int32_t* block_status,
                                                    int num_blocks,
                                                    int64_t num_tokens,
                                                    int num_topk,
                                                    int local_experts,
                                                    int tokens_per_block,
                                                    int window_blocks,
                                                    int threads,
                                                    int expand,
                                                    int64_t alignment,
                                                    const int32_t* packed_rank,
                                                    const int32_t* local_row,
                                                    int64_t* expert_counts,
                                                    int64_t* expert_offsets,
                                                    int64_t* send_counts,
                                                    int64_t* __restrict__ recv_rank_prefix,
                                                    const int64_t* totals,
                                                    int64_t* host_counts,
                                                    int32_t* __restrict__ recv_metadata,
                                                    int64_t* __restrict__ dst_slots,
                                                    int32_t* __restrict__ token_slots,
                                                    int64_t* __restrict__ slot_order,
                                                    int publisher,
                                                    const CountedToken<kCap>* own = nullptr) {
    extern __shared__ int32_t assign_lds[];
    __shared__ int64_t wave_padded[kMaxBlockTokens / kWave];
    __shared__ int64_t wave_assigned[kMaxBlockTokens / kWave];
    __shared__ int32_t wave_own[kMaxBlockTokens / kWave];
    __shared__ int32_t wave_before[kMaxBlockTokens / kWave];
    __shared__ int32_t wave_window_before[kMaxBlockTokens / kWave];
    __shared__ int status_bits;
    __shared__ int own_assignments;
    const int rows = local_experts + 1;
    int32_t* column_total = assign_lds;         // [L+1] totals over all blocks (fused scan only)
    int32_t* slot_base = assign_lds + rows;     // [L+1] assignments before this block -> first slot per expert
    // [L+1] histogram of this block's window (window_blocks consecutive blocks: the unit the slot-order
    // list is ordered by) -> where an expert's run starts inside the window's part of the list
    int32_t* order_base = assign_lds + 2 * rows;
    int32_t* window_before = assign_lds + 3 * rows;  // [L+1] the window's assignments in the blocks before this one

    const int tid = threadIdx.x;
    const int block = blockIdx.x;
    const int64_t token = static_cast<int64_t>(block) * tokens_per_block + tid;
    const bool live = tid < tokens_per_block && token < num_tokens;
    // kOwnBlock: the count pass ran in this very workgroup (the batch is one block) and `own` holds
    // what this thread found there; nothing of it is read back from memory.  With no more histogram
    // rows than threads that goes for the histogram too: the block's counts are the totals, nothing
    // lies before the block, and its window is the block.
    const bool own_counts = kOwnBlock && rows <= threads;
    int row_in_block;
    int32_t packed[kCap];
    if (kOwnBlock) {
        row_in_block = own->row;
#pragma unroll
        for (int k = 0; k < kCap; ++k)
            packed[k] = own->packed[k];
    } else {
        row_in_block = live ? local_row[token] : -1;
        // fetched here, ahead of the scans, so that the round trip overlaps them
#pragma unroll
        for (int k = 0; k < kCap; ++k)
            packed[k] = live ? packed_rank[token * num_topk + (k < num_topk ? k : 0)] : -1;
    }

    // the publishing workgroup gathers the blocks' routing status; the first word a thread is fetched here, used
    // behind the histogram loads, so that its round trip is not a second one behind theirs
    int first_status = 0;
    if (kOwnBlock)
        first_status = tid == 0 ? own->bad : 0;
    else if (kFusedScan && block == publisher && tid < num_blocks)
        first_status = block_status[tid];
    if (own_counts) {
        if (tid < rows) {
            column_total[tid] = own->first_count;
            slot_base[tid] = 0;
            order_base[tid] = own->first_count;
            window_before[tid] = 0;
        }
    } else if (kFusedScan) {
        for (int i = tid; i < 4 * rows; i += threads)
            assign_lds[i] = 0;
        if (tid == 0) {
            status_bits = 0;
            own_assignments = 0;
        }
        __syncthreads();
        const int window_first = block / window_blocks * window_blocks;
        const int window_end = window_first + window_blocks;

        const int columns_per_pass = rows < threads ? rows : threads;
        const int segments = threads / columns_per_pass;
        const int blocks_per_segment = (num_blocks + segments - 1) / segments;
        const int column_local = tid % columns_per_pass;
        const int segment = tid / columns_per_pass;
        const int begin = segment * blocks_per_segment;
        const int end = begin + blocks_per_segment < num_blocks ? begin + blocks_per_segment : num_blocks;
        // two columns a pass: with one more column than threads (L a multiple of the workgroup
        // size, plus the received-token column) the loads of both are in flight together
        for (int column0 = 0; column0 < rows; column0 += 2 * columns_per_pass) {
            const int column = column0 + column_local;
            const int second = column + columns_per_pass;
            const bool active = segment < segments && column < rows;
            const bool active_second = segment < segments && second < rows;
            int total[2] = {0, 0}, before[2] = {0, 0}, own[2] = {0, 0}, window[2] = {0, 0}, earlier[2] = {0, 0};
            // Histogram words are fetched sixteen blocks at a time, all loads of a batch in flight
            // together whatever the number of blocks (positions past the last block re-read it and
            // count nothing), and only a wavefront that holds a second column fetches it.
            const bool wave_has_second = column - (tid & (kWave - 1)) + columns_per_pass < rows;
            const int64_t second_or_first = active_second ? second : column;
            if (active) {
                for (int b0 = begin; b0 < end; b0 += 16) {
                    int fetched[16], fetched_second[16];
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int64_t b = b0 + j < end ? b0 + j : end - 1;
                        fetched[j] = block_counts[b * rows + column];
                    }
                    if (wave_has_second) {
#pragma unroll
                        for (int j = 0; j < 16; ++j) {
                            const int64_t b = b0 + j < end ? b0 + j : end - 1;
                            fetched_second[j] = block_counts[b * rows + second_or_first];
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int b = b0 + j;
                        const int count = b < end ? fetched[j] : 0;
                        const int count_second = wave_has_second && active_second && b < end ? fetched_second[j] : 0;
                        const bool in_window = b >= window_first && b < window_end;
                        total[0] += count;
                        total[1] += count_second;
                        before[0] += b < block ? count : 0;
                        before[1] += b < block ? count_second : 0;
                        own[0] = b == block ? count : own[0];
                        own[1] = b == block ? count_second : own[1];
                        window[0] += in_window ? count : 0;
                        window[1] += in_window ? count_second : 0;
                        earlier[0] += in_window && b < block ? count : 0;
                        earlier[1] += in_window && b < block ? count_second : 0;
                    }
                }
            }
            for (int i = 0; i < 2; ++i) {
                const int at = i == 0 ? column : second;
                if (!(i == 0 ? active : active_second))
                    continue;
                if (segments == 1) {
                    column_total[at] = total[i];
                    slot_base[at] = before[i];
                    order_base[at] = window[i];
                    window_before[at] = earlier[i];
                } else {
                    atomicAdd(&column_total[at], total[i]);
                    atomicAdd(&slot_base[at], before[i]);
                    if (window[i] != 0)
                        atomicAdd(&order_base[at], window[i]);
                    if (earlier[i] != 0)
                        atomicAdd(&window_before[at], earlier[i]);
                }
            }
            // this block's own assignments: one LDS atomic a wavefront (256 lanes adding to one word
            // one after the other were most of a microsecond in front of the barrier)
            int own_sum = (active && column < local_experts ? own[0] : 0) + (active_second && second < local_experts ? own[1] : 0);
#pragma unroll
            for (int distance = kWave / 2; distance > 0; distance /= 2)
                own_sum += __shfl_xor(own_sum, distance, kWave);
            if ((tid & (kWave - 1)) == 0 && own_sum != 0)
                atomicAdd(&own_assignments, own_sum);
        }
        if (block == publisher) {
            int bad = first_status;
            for (int b = tid + threads; b < num_blocks; b += threads)
                bad |= block_status[b];
            if (bad)
                atomicOr(&status_bits, bad);
        }
    } else {
        const int32_t* mine = block_counts + static_cast<int64_t>(block) * rows;
        const bool last_block = block + 1 >= num_blocks;
        for (int column = tid; column < rows; column += threads) {
            const int32_t before = mine[column];
            int32_t next;
            if (!last_block)
                next = mine[rows + column];
            else
                next = static_cast<int32_t>(column < local_experts ? expert_counts[column] : send_counts[0]);
            order_base[column] = next - before;
            window_before[column] = 0;  // the window is this block alone
            slot_base[column] = before;
        }
    }
    __syncthreads();

    const int per_thread = (local_experts + threads - 1) / threads;
    const int first = tid * per_thread < local_experts ? tid * per_thread : local_experts;
    const int last = first + per_thread < local_experts ? first + per_thread : local_experts;
    int64_t padded_sum = 0, count_sum = 0;
    int own_sum = 0, before_sum = 0, window_before_sum = 0;  // own_sum: the window's assignments (see order_base)
    for (int e = first; e < last; ++e) {
        if (kFusedScan) {
            const int64_t count = column_total[e];
            count_sum += count;
            padded_sum += round_up_to(count, alignment);
        }
        own_sum += order_base[e];
        before_sum += slot_base[e];
        window_before_sum += window_before[e];
    }
    const int64_t padded_scan = kFusedScan ? wave_inclusive_scan(padded_sum) : 0;
    const int64_t assigned_scan = kFusedScan ? wave_inclusive_scan(count_sum) : 0;
    const int own_scan = static_cast<int>(wave_inclusive_scan(own_sum));
    const int before_scan = static_cast<int>(wave_inclusive_scan(before_sum));
    const int window_before_scan = static_cast<int>(wave_inclusive_scan(window_before_sum));
    const int wave = tid / kWave;
    const int waves = threads / kWave;
    if ((tid & (kWave - 1)) == kWave - 1) {
        wave_padded[wave] = padded_scan;
        wave_assigned[wave] = assigned_scan;
        wave_own[wave] = own_scan;
        wave_before[wave] = before_scan;
        wave_window_before[wave] = window_before_scan;
    }
    __syncthreads();
    int64_t running = padded_scan - padded_sum;
    int running_own = own_scan - own_sum;
    int64_t capacity = 0, assigned = 0;
    // the window's assignments, those of all blocks before this one, and the window's share of the latter
    int window_total = 0, assigned_before = 0, window_earlier = 0;
    for (int w = 0; w < waves; ++w) {
        running += w < wave ? wave_padded[w] : 0;
        running_own += w < wave ? wave_own[w] : 0;
        capacity += wave_padded[w];
        assigned += wave_assigned[w];
        window_total += wave_own[w];
        assigned_before += wave_before[w];
        window_earlier += wave_window_before[w];
    }
    // this block's own assignments: the window's when the window is the block
    const int own_total = kFusedScan && !own_counts ? own_assignments : window_total;
    if (!kFusedScan)
        assigned = totals[0];
    for (int e = first; e < last; ++e) {
        if (kFusedScan) {
            const int64_t count = column_total[e];
            if (block == publisher) {
                expert_counts[e] = count;
                expert_offsets[e] = running;
            }
            slot_base[e] += static_cast<int32_t>(running);
            running += round_up_to(count, alignment);
        } else {
            slot_base[e] += static_cast<int32_t>(expert_offsets[e]);
        }
        const int in_window = order_base[e];
        order_base[e] = running_own + window_before[e];  // behind the expert's entries of the window's earlier blocks
        running_own += in_window;
    }
    const int64_t received = kFusedScan ? column_total[local_experts] : 0;
    __syncthreads();
    if (kFusedScan && block == publisher && tid == 0) {
        // Behind the workgroup's last barrier: the store to host memory and the wait that orders it
        // hold up one wavefront, not the whole workgroup (in front of the barrier they were a
        // microsecond of the kernel).
        expert_offsets[local_experts] = capacity;
        send_counts[0] = received;
        recv_rank_prefix[0] = received;
        host_counts[1] = capacity;
        host_counts[2] = assigned;
        host_counts[3] = kOwnBlock ? own->bad : status_bits;
        __threadfence_system();
        __hip_atomic_store(&host_counts[0], received, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    // The list is dense: a window's part starts where the assignments of the blocks before the window
    // end.  Every block also clears as many entries of the unused tail as it has masked choices.
    int64_t* order = nullptr;
    if (slot_order != nullptr) {
        order = slot_order + (assigned_before - window_earlier);
        // every block before the last one is full; the last one holds what is left of the batch
        const int64_t block_entries = static_cast<int64_t>(tokens_per_block) * num_topk;
        const int64_t tokens_left = num_tokens - static_cast<int64_t>(block) * tokens_per_block;
        const int64_t own_entries = (tokens_left < tokens_per_block ? tokens_left : tokens_per_block) * num_topk;
        int64_t* tail = slot_order + assigned + (block * block_entries - assigned_before);
        const int holes = static_cast<int>(own_entries) - own_total;
        for (int i = tid; i < holes; i += threads)
            tail[i] = -1;
        // The buffer's size does not depend on the block size: (T rounded up to 256) * K entries, then
        // the count word.  The last block (the one with the fewest tokens) clears what lies behind
        // the blocks' own entries, so that everything from entry A to the count word reads -1.
        const int64_t capacity_entries = (num_tokens + kMaxBlockTokens - 1) / kMaxBlockTokens * kMaxBlockTokens * num_topk;
        if (block == num_blocks - 1)
            for (int64_t i = num_tokens * num_topk + tid; i < capacity_entries; i += threads)
                slot_order[i] = -1;
        if (block == (kFusedScan ? publisher : 0) && tid == 0)
            slot_order[capacity_entries] = assigned;
    }
    if (live)
        assign_token_slots<kCap>(token, num_topk, expand, row_in_block, slot_base[local_experts], slot_base, order_base,
                                 packed, recv_metadata, dst_slots, token_slots, order);
}

template <int kCap, bool kFusedScan>
__global__ void __launch_bounds__(kMaxBlockTokens) layout_assign_kernel(const int32_t* __restrict__ block_counts,
                                                            const int32_t* __restrict__ block_status,
                                                            int num_blocks,
                                                            int64_t num_tokens,
                                                            int num_topk,
                                                            int local_experts,
                                                            int tokens_per_block,
                                                            int window_blocks,
                                                            int threads,
                                                            int expand,
                                                            int64_t alignment,
                                                            const int32_t* __restrict__ packed_rank,
                                                            const int32_t* __restrict__ local_row,
                                                            int64_t* expert_counts,
                                                            int64_t* expert_offsets,
                                                            int64_t* send_counts,
                                                            int64_t* recv_rank_prefix,
                                                            const int64_t* __restrict__ totals,
                                                            int64_t* host_counts,
                                                            int32_t* recv_metadata,
                                                            int64_t* dst_slots,
                                                            int32_t* token_slots,
                                                            int64_t* slot_order,
                                                            int publisher) {
    layout_assign_block<kCap, kFusedScan>(block_counts, block_status, num_blocks, num_tokens, num_topk, local_experts,
                                          tokens_per_block, window_blocks, threads, expand, alignment, packed_rank, local_row, expert_counts,
                                          expert_offsets, send_counts, recv_rank_prefix, totals, host_counts, recv_metadata,
                                          dst_slots, token_slots, slot_order, publisher);
}

// Whole layout in one launch when all tokens fit one block: the count pass, then (its results are
// this workgroup's own global writes: the barrier orders them for the workgroup, and a fence of
// wider scope in front of it would write the XCD's L2 back for nobody) the assignment pass.
template <int kCap>
__global__ void __launch_bounds__(kMaxBlockTokens) layout_single_block_kernel(const int64_t* topk_idx,
                                                                  int64_t num_tokens,
                                                                  int num_topk,
                                                                  int local_experts,
                                                                  int words,
                                                                  int threads,
                                                                  int expand,
                                                                  int64_t alignment,
                                                                  int64_t* snapshot,
                                                                  int32_t* block_counts,
                                                                  int32_t* block_status,
                                                                  int32_t* packed_rank,
                                                                  int32_t* local_row,
                                                                  int64_t* expert_counts,
                                                                  int64_t* expert_offsets,
                                                                  int64_t* send_counts,
                                                                  int64_t* recv_rank_prefix,
                                                                  int64_t* host_counts,
                                                                  int32_t* recv_metadata,
                                                                  int64_t* dst_slots,
                                                                  int32_t* token_slots,
                                                                  int64_t* slot_order) {
    CountedToken<kCap> counted;
    layout_count_block<kCap>(topk_idx, num_tokens, num_topk, local_experts, words, threads, snapshot, block_counts,
                             block_status, packed_rank, local_row, counted);
    __syncthreads();
    layout_assign_block<kCap, true, true>(block_counts, block_status, 1, num_tokens, num_topk, local_experts, words * 32, 1, threads,
                                          expand, alignment, packed_rank, local_row, expert_counts, expert_offsets, send_counts,
                                          recv_rank_prefix, nullptr, host_counts, recv_metadata, dst_slots, token_slots, slot_order, 0,
                                          &counted);
}


// Argument checks shared by the two layout entry points (everything but the workspace).
int check_layout_arguments(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts, int64_t alignment,
                           int expand, int hidden, const int32_t* recv_metadata, const int64_t* expert_counts,
                           const int64_t* expert_offsets, const int64_t* dst_slots, const int64_t* send_counts,
                           const int64_t* topk_snapshot, const int64_t* recv_rank_prefix, const int64_t* slot_order,
                           const int64_t* host_counts, const Knobs& knobs) {
    if (num_tokens < 0 || num_tokens > INT32_MAX || num_topk <= 0 || num_topk > kMaxTopk || num_local_experts <= 0 ||
        num_local_experts >= (int64_t{1} << (31 - kRankBits)) || alignment <= 0 || alignment > (int64_t{1} << 31) || hidden < 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (expert_counts == nullptr || expert_offsets == nullptr || send_counts == nullptr || recv_rank_prefix == nullptr ||
        host_counts == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (num_tokens > 0 && (topk_idx == nullptr || recv_metadata == nullptr || dst_slots == nullptr || topk_snapshot == nullptr))
        return NANOEP_ERR_INVALID_ARGUMENT;
    // the slot-order list packs token * K + k into 32 bits and only exists for the expanded layout
    if (slot_order != nullptr && (!expand || num_tokens * num_topk >= (int64_t{1} << 31)))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (layout_tokens_per_block(num_tokens, num_local_experts, hidden, knobs) == 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    return NANOEP_OK;
}

// Enqueues the layout launches over a carved workspace; the arguments have been checked.
int enqueue_layout(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts, int64_t alignment,
                   int expand, int hidden, int32_t* recv_metadata, int64_t* expert_counts, int64_t* expert_offsets,
                   int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot, int64_t* recv_rank_prefix,
                   int32_t* token_slots, int64_t* slot_order, const LayoutWorkspace& ws, int64_t* host_counts,
                   void* stream_handle, const Knobs& knobs) {
    const int tokens_per_block = layout_tokens_per_block(num_tokens, num_local_experts, hidden, knobs);
    const int64_t blocks64 = (num_tokens + tokens_per_block - 1) / tokens_per_block;
    const int blocks = static_cast<int>(blocks64);
    const int experts = static_cast<int>(num_local_experts);
    const int words = tokens_per_block / 32;
    auto stream = static_cast<hipStream_t>(stream_handle);

    __atomic_store_n(&host_counts[0], int64_t{-1}, __ATOMIC_RELEASE);
    // whole wavefronts: the kernels' scans take a wavefront's sums from its last lane (a forced window of
    // 96, 160 or 224 tokens would otherwise leave the experts of a trailing half wavefront out)
    const int count_threads = (tokens_per_block + kWave - 1) / kWave * kWave;
    // Two launches while every block can afford to sum the block histograms itself (blocks x (L+1)
    // loads from L2, spread over the workgroup): measured faster than the single-workgroup scan up to
    // 1024 blocks whatever the expert count (8192 tokens, 256 experts: 21 against 27 us; 262144
    // tokens: 159 against 198 us).  Beyond, the blocks^2 loads lose (2^20 tokens, 8 experts: 124
    // against 67 us) and a third launch does the scan once.
    const bool fused_scan = layout_uses_fused_scan(num_tokens, num_local_experts, hidden, knobs);
    const int forced_launches = knobs.layout_launches;
    const int window_blocks = layout_window_blocks(num_tokens, num_local_experts, hidden, fused_scan, knobs);
    hipError_t launch_status = hipSuccess;
    with_topk_cap(num_topk, [&](auto cap) {
        constexpr int kCap = decltype(cap)::value;
        if (blocks == 1 && forced_launches == 0) {
            const size_t count_lds = static_cast<size_t>(experts + 1) * (words * 6 + 4);
            const size_t assign_lds = static_cast<size_t>(experts + 1) * 16;
            layout_single_block_kernel<kCap><<<1, count_threads, count_lds > assign_lds ? count_lds : assign_lds, stream>>>(
                topk_idx, num_tokens, num_topk, experts, words, count_threads, expand, alignment, topk_snapshot,
                ws.block_counts, ws.block_status, ws.packed_rank, ws.local_row, expert_counts, expert_offsets, send_counts,
                recv_rank_prefix, host_counts, recv_metadata, dst_slots, token_slots, slot_order);
            launch_status = hipGetLastError();
            return;
        }
        if (blocks > 0) {
            const size_t lds = static_cast<size_t>(experts + 1) * (words * 6 + 4);
            layout_count_kernel<kCap><<<blocks, count_threads, lds, stream>>>(
                topk_idx, num_tokens, num_topk, experts, words, count_threads, topk_snapshot, ws.block_counts,
                ws.block_status, ws.packed_rank, ws.local_row);
            if ((launch_status = hipGetLastError()) != hipSuccess)
                return;
        }
        const size_t assign_lds = static_cast<size_t>(experts + 1) * 16;
        if (fused_scan) {
            // one workgroup more than there are blocks: the publisher
            layout_assign_kernel<kCap, true><<<blocks + 1, count_threads, assign_lds, stream>>>(
                ws.block_counts, ws.block_status, blocks, num_tokens, num_topk, experts, tokens_per_block, window_blocks,
                count_threads, expand, alignment, ws.packed_rank, ws.local_row, expert_counts, expert_offsets, send_counts,
                recv_rank_prefix, ws.totals, host_counts, recv_metadata, dst_slots, token_slots, slot_order, blocks);
            launch_status = hipGetLastError();
            return;
        }
        layout_scan_kernel<<<1, kScanThreads, static_cast<size_t>(experts + 1) * 4, stream>>>(
            ws.block_counts, ws.block_status, blocks, experts, alignment, expert_counts, expert_offsets, send_counts,
            recv_rank_prefix, ws.totals, host_counts);
        if ((launch_status = hipGetLastError()) != hipSuccess)
            return;
        if (blocks > 0) {
            layout_assign_kernel<kCap, false><<<blocks, count_threads, assign_lds, stream>>>(
                ws.block_counts, ws.block_status, blocks, num_tokens, num_topk, experts, tokens_per_block, 1, count_threads,
                expand, alignment, ws.packed_rank, ws.local_row, expert_counts, expert_offsets, send_counts,
                recv_rank_prefix, ws.totals, host_counts, recv_metadata, dst_slots, token_slots, slot_order, 0);
            launch_status = hipGetLastError();
        }
    });
    NANOEP_HIP_TRY(launch_status);
    return NANOEP_OK;
}

// ---- The private handle tensors rebuilt from a handle's own public ones -------------------------
//
// A handle that went through a caller keeping only the reference's seven tensors has lost the slot
// table and the slot-order list.  Both are functions of dst_slots and recv_metadata alone:
// token_slots[t][k] = recv_metadata[dst_slots[t]][2 + k] (-1 when the token was not sent or the slot
// lies outside [0, C)), and the list is, window of consecutive tokens by window, the valid (slot,
// t * K + k) pairs in ascending slot order.  Nothing here looks at the routing ids or assumes the
// slots were made by this library: the handle is followed as it is written.

// Largest number of list entries one window may hold here: the sort runs in LDS, 8 bytes an entry.
constexpr int kRebuildMaxWindowEntries = 4096;
constexpr int kRebuildThreads = 1024;

// Tokens of one window of a rebuilt list: the layout's own choice for this batch, halved until a
// window's T * K entries fit the sort.
int rebuild_window_tokens(int64_t tokens_total, int num_topk, int hidden, const Knobs& knobs) {
    int window = layout_window_tokens(tokens_total, hidden, knobs);
    if (window > kMaxWindowTokens)
        window = kMaxWindowTokens;
    while (window > 32 && static_cast<int64_t>(window) * num_topk > kRebuildMaxWindowEntries)
        window /= 2;
    return window;
}

// One workgroup per window: the slot table of the window's tokens and the number of valid entries.
__global__ void __launch_bounds__(kRebuildThreads) rebuild_table_kernel(const int32_t* __restrict__ recv_metadata,  // [N][K+2]
                                                                       const int64_t* __restrict__ dst_slots,     // [T]
                                                                       int64_t recv_count,
                                                                       int64_t out_rows,
                                                                       int64_t num_tokens,
                                                                       int num_topk,
                                                                       int window_tokens,
                                                                       int32_t* __restrict__ token_slots,  // [T][K]
                                                                       int32_t* __restrict__ window_counts) {
    __shared__ int valid_entries;
    if (threadIdx.x == 0)
        valid_entries = 0;
    __syncthreads();
    const int64_t first = static_cast<int64_t>(blockIdx.x) * window_tokens * num_topk;
    const int64_t batch_end = num_tokens * num_topk;
    const int64_t window_end = first + static_cast<int64_t>(window_tokens) * num_topk;
    const int64_t end = window_end < batch_end ? window_end : batch_end;
    int mine = 0;
    for (int64_t flat = first + threadIdx.x; flat < end; flat += kRebuildThreads) {
        const int64_t token = flat / num_topk;
        const int k = static_cast<int>(flat - token * num_topk);
        const int64_t row = dst_slots[token];
        int32_t slot = -1;
        if (row >= 0 && row < recv_count)
            slot = recv_metadata[row * (num_topk + 2) + 2 + k];
        if (slot < 0 || slot >= out_rows)
            slot = -1;
        token_slots[flat] = slot;
        mine += slot >= 0;
    }
#pragma unroll
    for (int distance = kWave / 2; distance > 0; distance /= 2)
        mine += __shfl_xor(mine, distance, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && mine != 0)
        atomicAdd(&valid_entries, mine);
    __syncthreads();
    if (threadIdx.x == 0)
        window_counts[blockIdx.x] = valid_entries;
}

// One workgroup per window: sorts the window's (slot, source) pairs in LDS (bitonic network over
// `sort_size` keys, a power of two; masked choices sort behind everything as the largest key) and
// writes the valid ones where the list has room for them: behind the entries of all earlier
// windows.  The rest of the buffer reads -1 up to the count word, as the layout leaves it.
__global__ void __launch_bounds__(kRebuildThreads) rebuild_order_kernel(const int32_t* __restrict__ token_slots,    // [T][K]
                                                                       const int32_t* __restrict__ window_counts,  // [windows]
                                                                       int64_t num_tokens,
                                                                       int num_topk,
                                                                       int window_tokens,
                                                                       int num_windows,
                                                                       int sort_size,
                                                                       int64_t* __restrict__ slot_order,
                                                                       int64_t capacity_entries,
                                                                       int64_t* host_count,  // pinned, or null
                                                                       int64_t host_tag) {
    extern __shared__ int64_t sort_keys[];
    __shared__ int64_t before_sum;
    __shared__ int64_t total_sum;
    const int window = blockIdx.x;
    const int tid = threadIdx.x;
    if (tid == 0) {
        before_sum = 0;
        total_sum = 0;
    }
    const int64_t first = static_cast<int64_t>(window) * window_tokens * num_topk;
    const int64_t batch_end = num_tokens * num_topk;
    const int64_t window_end = first + static_cast<int64_t>(window_tokens) * num_topk;
    const int64_t end = window_end < batch_end ? window_end : batch_end;
    for (int i = tid; i < sort_size; i += kRebuildThreads) {
        const int64_t flat = first + i;
        int64_t key = INT64_MAX;
        if (flat < end) {
            const int32_t slot = token_slots[flat];
            if (slot >= 0)
                key = (static_cast<int64_t>(slot) << 32) | static_cast<int64_t>(static_cast<uint32_t>(flat));
        }
        sort_keys[i] = key;
    }
    __syncthreads();
    // valid entries of the windows before this one, and of all windows
    int64_t before = 0, total = 0;
    for (int w = tid; w < num_windows; w += kRebuildThreads) {
        const int count = window_counts[w];
        total += count;
        before += w < window ? count : 0;
    }
#pragma unroll
    for (int distance = kWave / 2; distance > 0; distance /= 2) {
        before += __shfl_xor(before, distance, kWave);
        total += __shfl_xor(total, distance, kWave);
    }
    if ((tid & (kWave - 1)) == 0 && total != 0) {
        atomicAdd(reinterpret_cast<unsigned long long*>(&before_sum), static_cast<unsigned long long>(before));
        atomicAdd(reinterpret_cast<unsigned long long*>(&total_sum), static_cast<unsigned long long>(total));
    }
    for (int size = 2; size <= sort_size; size *= 2) {
        for (int stride = size / 2; stride > 0; stride /= 2) {
            for (int i = tid; i < sort_size; i += kRebuildThreads) {
                const int partner = i ^ stride;
                if (partner > i) {
                    const bool ascending = (i & size) == 0;
                    const int64_t a = sort_keys[i], b = sort_keys[partner];
                    if ((a > b) == ascending) {
                        sort_keys[i] = b;
                        sort_keys[partner] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
    __syncthreads();
    const int64_t assigned_before = before_sum;
    const int64_t assigned = total_sum;
    const int own = window_counts[window];
    for (int i = tid; i < own; i += kRebuildThreads)
        slot_order[assigned_before + i] = sort_keys[i];
    // the unused tail: every window clears as many entries as it has masked choices, the last one also
    // what lies between the batch's last choice and the count word
    const int64_t own_entries = end - first;
    int64_t* tail = slot_order + assigned + (first - assigned_before);
    for (int64_t i = tid; i < own_entries - own; i += kRebuildThreads)
        tail[i] = -1;
    if (window == num_windows - 1) {
        for (int64_t i = batch_end + tid; i < capacity_entries; i += kRebuildThreads)
            slot_order[i] = -1;
        if (tid == 0) {
            slot_order[capacity_entries] = assigned;
            if (host_count != nullptr) {
                __threadfence_system();
                __hip_atomic_store(host_count, host_tag | assigned, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
    }
}

// Address of this file's `scratch` array on the current device, resolved once per device (each GPU
// holds its own copy at its own address).
constexpr int kMaxDevices = 64;
std::mutex g_static_scratch_mutex;
void* g_static_scratch[kMaxDevices] = {};

int static_scratch_of_current_device(void** out) {
    int device = -1;
    NANOEP_HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices)
        return NANOEP_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch[device] == nullptr) {
        void* address = nullptr;
        NANOEP_HIP_TRY(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
        if (address == nullptr)
            return NANOEP_ERR_HIP;
        g_static_scratch[device] = address;
    }
    *out = g_static_scratch[device];
    return NANOEP_OK;
}

}  // namespace
}  // namespace nanoep

using namespace nanoep;

extern "C" {

size_t nanoep_layout_workspace_bytes(int64_t num_tokens, int num_topk, int64_t num_local_experts) {
    if (num_tokens < 0 || num_topk <= 0 || num_local_experts <= 0)
        return 0;
    return carve_layout_workspace(nullptr, num_tokens, num_topk, num_local_experts, current_knobs()).bytes;
}

int nanoep_layout_block_tokens(int64_t num_tokens, int64_t num_local_experts, int hidden) {
    if (num_local_experts <= 0 || num_tokens < 0 || hidden < 0)
        return 0;
    const Knobs knobs = current_knobs();
    // tokens the slot-order list is ordered by: the layout workgroup's tokens times the blocks of a window
    const int per_block = layout_tokens_per_block(num_tokens, num_local_experts, hidden, knobs);
    const bool fused = layout_uses_fused_scan(num_tokens, num_local_experts, hidden, knobs);
    return per_block * layout_window_blocks(num_tokens, num_local_experts, hidden, fused, knobs);
}

int64_t nanoep_slot_order_entries(int64_t num_tokens, int num_topk, int64_t num_local_experts) {
    if (num_tokens < 0 || num_topk <= 0 || num_local_experts <= 0)
        return 0;
    if (layout_smallest_block(num_tokens, num_local_experts, current_knobs()) == 0 || num_tokens == 0)
        return 0;
    // whole blocks of any size the layout may take, then the count word
    return (num_tokens + kMaxBlockTokens - 1) / kMaxBlockTokens * kMaxBlockTokens * num_topk + 1;
}

int nanoep_layout(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts,
                  int64_t alignment, int expand, int hidden, int32_t* recv_metadata, int64_t* expert_counts,
                  int64_t* expert_offsets, int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot,
                  int64_t* recv_rank_prefix, int32_t* token_slots, int64_t* slot_order, void* workspace,
                  size_t workspace_bytes, int64_t* host_counts, void* stream_handle) {
    const Knobs knobs = current_knobs();
    const int status = check_layout_arguments(topk_idx, num_tokens, num_topk, num_local_experts, alignment, expand, hidden,
                                              recv_metadata, expert_counts, expert_offsets, dst_slots, send_counts, topk_snapshot,
                                              recv_rank_prefix, slot_order, host_counts, knobs);
    if (status != NANOEP_OK)
        return status;
    if (workspace == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const LayoutWorkspace ws = carve_layout_workspace(workspace, num_tokens, num_topk, num_local_experts, knobs);
    if (ws.bytes > workspace_bytes)
        return NANOEP_ERR_WORKSPACE;
    return enqueue_layout(topk_idx, num_tokens, num_topk, num_local_experts, alignment, expand, hidden, recv_metadata, expert_counts,
                          expert_offsets, dst_slots, send_counts, topk_snapshot, recv_rank_prefix, token_slots, slot_order, ws,
                          host_counts, stream_handle, knobs);
}

int nanoep_layout_static(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts,
                         int64_t alignment, int expand, int hidden, int32_t* recv_metadata, int64_t* expert_counts,
                         int64_t* expert_offsets, int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot,
                         int64_t* recv_rank_prefix, int32_t* token_slots, int64_t* slot_order, int64_t* host_counts,
                         void* stream_handle) {
    const Knobs knobs = current_knobs();
    const int status = check_layout_arguments(topk_idx, num_tokens, num_topk, num_local_experts, alignment, expand, hidden,
                                              recv_metadata, expert_counts, expert_offsets, dst_slots, send_counts, topk_snapshot,
                                              recv_rank_prefix, slot_order, host_counts, knobs);
    if (status != NANOEP_OK)
        return status;
    // the size is checked before any device is touched
    if (carve_layout_workspace(nullptr, num_tokens, num_topk, num_local_experts, knobs).bytes > NANOEP_STATIC_SCRATCH_BYTES)
        return NANOEP_ERR_SCRATCH_LIMIT;
    void* base = nullptr;
    const int scratch_status = static_scratch_of_current_device(&base);
    if (scratch_status != NANOEP_OK)
        return scratch_status;
    // Nothing in the workspace has to start at zero: the count pass writes every histogram row, status
    // word, rank entry and receive row that the later passes of the same call read.
    const LayoutWorkspace ws = carve_layout_workspace(base, num_tokens, num_topk, num_local_experts, knobs);
    return enqueue_layout(topk_idx, num_tokens, num_topk, num_local_experts, alignment, expand, hidden, recv_metadata, expert_counts,
                          expert_offsets, dst_slots, send_counts, topk_snapshot, recv_rank_prefix, token_slots, slot_order, ws,
                          host_counts, stream_handle, knobs);
}

size_t nanoep_rebuild_workspace_bytes(int64_t num_tokens, int num_topk) {
    if (num_tokens < 0 || num_topk <= 0 || num_topk > kMaxTopk)
        return 0;
    // one int32 per window of the smallest size a rebuilt list takes
    return align_up(static_cast<size_t>((num_tokens + 31) / 32) * 4, 256) + 256;
}

int nanoep_rebuild_window_tokens(int64_t num_tokens, int num_topk, int hidden) {
    if (num_tokens < 0 || num_topk <= 0 || num_topk > kMaxTopk || hidden < 0)
        return 0;
    return rebuild_window_tokens(num_tokens, num_topk, hidden, current_knobs());
}

int nanoep_rebuild_order(const int32_t* recv_metadata, const int64_t* dst_slots, int64_t recv_count, int64_t expanded_capacity,
                         int64_t num_tokens, int num_topk, int64_t num_local_experts, int hidden, int32_t* token_slots,
                         int64_t* slot_order, void* workspace, size_t workspace_bytes, int64_t* host_count, int64_t host_tag,
                         void* stream_handle) {
    if (num_tokens <= 0 || num_tokens > INT32_MAX || num_topk <= 0 || num_topk > kMaxTopk || num_local_experts <= 0 || hidden < 0 ||
        recv_count < 0 || recv_count > num_tokens || expanded_capacity < 0 || expanded_capacity > INT32_MAX ||
        num_tokens * num_topk >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (dst_slots == nullptr || token_slots == nullptr || slot_order == nullptr || workspace == nullptr ||
        (recv_count > 0 && recv_metadata == nullptr) || host_tag < 0 || (host_tag & 0xffffffffll) != 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const Knobs knobs = current_knobs();
    if (layout_smallest_block(num_tokens, num_local_experts, knobs) == 0)
        return NANOEP_ERR_INVALID_ARGUMENT;  // no slot-order buffer exists for this geometry
    if (nanoep_rebuild_workspace_bytes(num_tokens, num_topk) > workspace_bytes)
        return NANOEP_ERR_WORKSPACE;
    const int window = rebuild_window_tokens(num_tokens, num_topk, hidden, knobs);
    const int64_t windows = (num_tokens + window - 1) / window;
    int sort_size = 2;
    while (sort_size < window * num_topk)
        sort_size *= 2;
    const int64_t capacity_entries = (num_tokens + kMaxBlockTokens - 1) / kMaxBlockTokens * kMaxBlockTokens * num_topk;
    auto* window_counts = static_cast<int32_t*>(workspace);
    auto stream = static_cast<hipStream_t>(stream_handle);
    if (host_count != nullptr)
        __atomic_store_n(host_count, int64_t{-1}, __ATOMIC_RELEASE);
    rebuild_table_kernel<<<static_cast<unsigned>(windows), kRebuildThreads, 0, stream>>>(
        recv_metadata, dst_slots, recv_count, expanded_capacity, num_tokens, num_topk, window, token_slots, window_counts);
    NANOEP_HIP_TRY(hipGetLastError());
    rebuild_order_kernel<<<static_cast<unsigned>(windows), kRebuildThreads, static_cast<size_t>(sort_size) * 8, stream>>>(
        token_slots, window_counts, num_tokens, num_topk, window, static_cast<int>(windows), sort_size, slot_order, capacity_entries,
        host_count, host_tag);
    NANOEP_HIP_TRY(hipGetLastError());
    return NANOEP_OK;
}

int nanoep_wait_counts(int64_t* host_counts, void* stream_handle, double timeout_seconds,
                       int64_t out[NANOEP_HOST_COUNT_WORDS]) {
    if (host_counts == nullptr || out == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    auto stream = static_cast<hipStream_t>(stream_handle);
    // The wait is a plain spin on the mailbox word: the counts usually arrive within microseconds,
    // and whoever waits for them wants to know at once.  The clock is read every 256 spins; the
    // stream is only asked how it is doing every 100 us of waiting (the question itself takes the
    // runtime microseconds, during which a published count would go unnoticed).
    timespec start{};
    clock_gettime(CLOCK_MONOTONIC, &start);
    double next_stream_check = 100e-6;
    uint64_t spins = 0;
    while (true) {
        const int64_t received = __atomic_load_n(&host_counts[0], __ATOMIC_ACQUIRE);
        if (received >= 0)
            break;
        if ((++spins & 0xff) == 0) {
            // the clock first: a caller with no patience left is answered without touching the stream
            timespec now{};
            clock_gettime(CLOCK_MONOTONIC, &now);
            const double elapsed = (now.tv_sec - start.tv_sec) + 1e-9 * (now.tv_nsec - start.tv_nsec);
            if (elapsed > timeout_seconds) {
                // a last look at the mailbox, and at a stream that may have failed rather than stalled
                if (__atomic_load_n(&host_counts[0], __ATOMIC_ACQUIRE) >= 0)
                    break;
                if (stream != nullptr) {
                    const hipError_t state = hipStreamQuery(stream);
                    if (state != hipSuccess && state != hipErrorNotReady) {
                        g_last_hip_error = state;
                        return NANOEP_ERR_HIP;
                    }
                }
                return NANOEP_ERR_TIMEOUT;
            }
            if (elapsed < next_stream_check)
                continue;
            next_stream_check = elapsed + 100e-6;
            // A finished (or failed) stream with no published count means the layout never ran.
            const hipError_t state = hipStreamQuery(stream);
            if (state != hipErrorNotReady) {
                if (state != hipSuccess) {
                    g_last_hip_error = state;
                    return NANOEP_ERR_HIP;
                }
                if (__atomic_load_n(&host_counts[0], __ATOMIC_ACQUIRE) >= 0)
                    break;
                return NANOEP_ERR_TIMEOUT;
            }
        }
    }
    for (int i = 0; i < NANOEP_HOST_COUNT_WORDS; ++i)
        out[i] = __atomic_load_n(&host_counts[i], __ATOMIC_RELAXED);
    return out[3] != 0 ? NANOEP_ERR_ROUTING : NANOEP_OK;
}

}  // extern "C"
