// MI355X (gfx950, wave64) kernels for one rank's expert-parallel dispatch / combine, and the
// C ABI declared in include/nanoep_hip.h.
//
// Data layout in HBM (all row-major, contiguous):
//   x, recv_x, y, out_x, bias : bf16 rows of H elements, moved as 16-byte vectors (H/8 per row)
//   topk_idx / snapshot       : int64 [T,K]
//   recv_metadata             : int32 [N,K+2]   (src_rank, src_token, K values)
//   weights                   : fp32 [T,K] at the source, [N,K] compact, [C] expanded
//
// Kernels
//   layout_count_kernel  : one workgroup per block of tokens; LDS bit matrix (expert x token) built
//                          with LDS atomics, popcount prefixes give the in-block stable rank of
//                          every (token,k) and the block's per-expert histogram.
//   layout_assign_kernel<fused scan> : (few blocks) every workgroup sums the block histograms into
//                          LDS, scans the aligned expert totals and writes its tokens' part of the
//                          handle and of the slot-order list; workgroup 0 publishes N, C to the host.
//   layout_single_block_kernel : (one block) count and assignment passes in a single launch.
//   layout_scan_kernel + layout_assign_kernel<no scan> : (many blocks) the same in two launches, one
//                          workgroup doing the scans: slot = offset[e] + block_base[b][e] + rank.
//   dispatch_ordered_kernel : expanded layouts with the layout's slot-order list: one wavefront per
//                          (list entry, row chunk), token block by token block and expert-major
//                          inside a block, so a block's source rows stay in one XCD's L2 and every
//                          expert receives runs of consecutive rows; one 128-bit load and one
//                          nontemporal 128-bit store per lane.
//   dispatch_rows_kernel : the same work item walked in source-token order (small batches, handles
//                          without the list); extra work items zero-fill the alignment gaps.
//   dispatch_compact_kernel / combine_compact_kernel : compact layouts are row copies with holes;
//                          plain launch order, single-wavefront workgroups, nothing but the copy.
//   combine_rows_kernel  : one wavefront per (source token, row chunk): gathers the token's rows in
//                          ascending k, fp32 accumulate, one round-to-nearest-even bf16 store.
//   combine_few_rows_kernel : the same for K <= 4 with the slot table, without the bookkeeping.
//
// Every byte moved is HBM-bound integer/byte work; there is no contraction, hence no MFMA.

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <type_traits>

#include "nanoep_hip.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWave * kWavesPerBlock;
constexpr int kScanThreads = 1024;
constexpr int kMaxTopk = 32;
constexpr size_t kLayoutLdsBudget = 60 * 1024;

thread_local hipError_t g_last_hip_error = hipSuccess;

#define NANOEP_HIP_TRY(expr)              \
    do {                                  \
        const hipError_t status_ = (expr); \
        if (status_ != hipSuccess) {      \
            g_last_hip_error = status_;   \
            return NANOEP_ERR_HIP;        \
        }                                 \
    } while (0)

inline size_t align_up(size_t value, size_t alignment) { return (value + alignment - 1) / alignment * alignment; }

int env_int(const char* name, int fallback) {
    const char* text = std::getenv(name);
    if (text == nullptr || *text == '\0')
        return fallback;
    return std::atoi(text);
}

// Calls f with the smallest compile-time bound in {4, 8, 16, 32} that covers num_topk.
template <typename F>
void with_topk_cap(int num_topk, F&& f) {
    if (num_topk <= 4)
        f(std::integral_constant<int, 4>{});
    else if (num_topk <= 8)
        f(std::integral_constant<int, 8>{});
    else if (num_topk <= 16)
        f(std::integral_constant<int, 16>{});
    else
        f(std::integral_constant<int, 32>{});
}

// ---------------------------------------------------------------------------------------------
// Routing layout
// ---------------------------------------------------------------------------------------------

// Tokens handled by one layout workgroup: the LDS bit matrix has (L+1) rows of tokens/32 words
// plus a 16-bit prefix per word, so the block shrinks as the expert count grows.
int layout_tokens_per_block(int64_t local_experts) {
    if (static_cast<size_t>(local_experts + 1) * 12 > kLayoutLdsBudget)  // three int32 arrays of the assignment kernel
        return 0;
    for (int tokens = 256; tokens >= 32; tokens /= 2) {
        const size_t words = static_cast<size_t>(tokens / 32);
        if (static_cast<size_t>(local_experts + 1) * (words * 6 + 4) <= kLayoutLdsBudget)
            return tokens;
    }
    return 0;
}

struct LayoutWorkspace {
    int32_t* block_counts;  // [NB][L+1]; column L counts tokens with any valid choice
    int32_t* block_status;  // [NB]
    int32_t* packed_rank;   // [T][K]  (expert << 8) | in-block rank, or -1
    int32_t* local_row;     // [T]
    int64_t* totals;        // [1] total assignments, handed from the scan kernel to the assignment kernel
    size_t bytes;
};

LayoutWorkspace carve_layout_workspace(void* base, int64_t tokens, int topk, int64_t local_experts) {
    const int per_block = layout_tokens_per_block(local_experts);
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
constexpr int kRankMask = (1 << kRankBits) - 1;

// One thread per token.  bits[e][w] has bit (token & 31) of word (token >> 5) set when the token
// chose expert e; row L marks tokens with any valid choice.  Experts inside a token are distinct,
// so the order of one expert's assignments is the token order and a popcount prefix is the rank.
// The token's routing ids are fetched in one batch of independent loads (kCap >= K of them, the
// surplus re-reads id 0) and stay in registers for both passes over the bit matrix.
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
                                                   int32_t* local_row) {
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

    int64_t raw[kCap];
    const int64_t* mine = topk_idx + (live ? token : 0) * num_topk;
#pragma unroll
    for (int k = 0; k < kCap; ++k)
        raw[k] = mine[k < num_topk ? k : 0];

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
        else
            snapshot[token * num_topk + k] = expert;
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

    for (int row = threadIdx.x; row < rows; row += threads) {
        int running = 0;
        for (int w = 0; w < words; ++w) {
            prefix[static_cast<size_t>(row) * words + w] = static_cast<uint16_t>(running);
            running += __popc(bits[static_cast<size_t>(row) * stride + w]);
        }
        block_counts[static_cast<int64_t>(blockIdx.x) * rows + row] = running;
    }
    if (threadIdx.x == 0)
        block_status[blockIdx.x] = block_bad;
    __syncthreads();

    if (live) {
        const uint32_t below = bit - 1;
#pragma unroll
        for (int k = 0; k < kCap; ++k) {
            const int id = ids[k];
            int32_t packed = -1;
            if (id >= 0) {
                const int rank = prefix[static_cast<size_t>(id) * words + word] +
                                 __popc(bits[static_cast<size_t>(id) * stride + word] & below);
                packed = (id << kRankBits) | rank;
            }
            if (k < num_topk)
                packed_rank[token * num_topk + k] = packed;
        }
        const uint32_t received = bits[static_cast<size_t>(local_experts) * stride + word];
        local_row[token] = (received & bit) ? prefix[static_cast<size_t>(local_experts) * words + word] + __popc(received & below) : -1;
    }
}

template <int kCap>
__global__ void __launch_bounds__(256) layout_count_kernel(const int64_t* __restrict__ topk_idx,
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
    layout_count_block<kCap>(topk_idx, num_tokens, num_topk, local_experts, words, threads, snapshot, block_counts,
                             block_status, packed_rank, local_row);
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

// Writes one token's part of the handle.  `slot_base[e]` is the first slot of this block's
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
                                                   const int32_t* __restrict__ packed_rank,
                                                   int32_t* __restrict__ recv_metadata,
                                                   int64_t* __restrict__ dst_slots,
                                                   int32_t* __restrict__ token_slots,
                                                   int64_t* __restrict__ order) {
    int32_t packed[kCap];
#pragma unroll
    for (int k = 0; k < kCap; ++k)
        packed[k] = packed_rank[token * num_topk + (k < num_topk ? k : 0)];
    if (row_in_block < 0) {
        dst_slots[token] = -1;
        if (token_slots != nullptr)
            for (int k = 0; k < num_topk; ++k)
                token_slots[token * num_topk + k] = -1;
        return;
    }
    const int64_t row = row_base + row_in_block;
    dst_slots[token] = row;
    int32_t* out = recv_metadata + row * (num_topk + 2);
    out[0] = 0;
    out[1] = static_cast<int32_t>(token);
#pragma unroll
    for (int k = 0; k < kCap; ++k) {
        if (k >= num_topk)
            break;
        int32_t value = -1;
        if (packed[k] >= 0) {
            const int expert = packed[k] >> kRankBits;
            const int rank = packed[k] & kRankMask;
            value = expand ? slot_base[expert] + rank : expert;
            if (order != nullptr) {
                const uint32_t source = static_cast<uint32_t>(token * num_topk + k);
                order[order_base[expert] + rank] = (static_cast<int64_t>(value) << 32) | source;
            }
        }
        out[2 + k] = value;
        if (token_slots != nullptr)
            token_slots[token * num_topk + k] = value;
    }
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
// own, then the aligned exclusive scan over experts, all in LDS; workgroup 0 also writes the
// per-expert outputs and the host mailbox (word 0 last).  Otherwise layout_scan_kernel has done
// that and `block_counts` holds each block's exclusive prefixes.
//
// Either way the workgroup also scans its own histogram over experts: that places every
// assignment of the block in expert-major order inside the block's run of `slot_order`; the runs
// of consecutive blocks follow each other without gaps and the unused tail of the list is -1.
template <int kCap, bool kFusedScan>
__device__ __forceinline__ void layout_assign_block(const int32_t* block_counts,
                                                    const int32_t* block_status,
                                                    int num_blocks,
                                                    int64_t num_tokens,
                                                    int num_topk,
                                                    int local_experts,
                                                    int tokens_per_block,
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
                                                    int64_t* __restrict__ slot_order) {
    extern __shared__ int32_t assign_lds[];
    __shared__ int64_t wave_padded[kWavesPerBlock];
    __shared__ int64_t wave_assigned[kWavesPerBlock];
    __shared__ int32_t wave_own[kWavesPerBlock];
    __shared__ int32_t wave_before[kWavesPerBlock];
    __shared__ int status_bits;
    const int rows = local_experts + 1;
    int32_t* column_total = assign_lds;         // [L+1] totals over all blocks (fused scan only)
    int32_t* slot_base = assign_lds + rows;     // [L+1] assignments before this block -> first slot per expert
    int32_t* order_base = assign_lds + 2 * rows;  // [L+1] this block's histogram -> its exclusive scan

    const int tid = threadIdx.x;
    const int block = blockIdx.x;
    const int64_t token = static_cast<int64_t>(block) * tokens_per_block + tid;
    const bool live = tid < tokens_per_block && token < num_tokens;
    const int row_in_block = live ? local_row[token] : -1;

    if (kFusedScan) {
        for (int i = tid; i < 2 * rows; i += threads)
            assign_lds[i] = 0;
        if (tid == 0)
            status_bits = 0;
        __syncthreads();

        const int columns_per_pass = rows < threads ? rows : threads;
        const int segments = threads / columns_per_pass;
        const int blocks_per_segment = (num_blocks + segments - 1) / segments;
        const int column_local = tid % columns_per_pass;
        const int segment = tid / columns_per_pass;
        const int begin = segment * blocks_per_segment;
        const int end = begin + blocks_per_segment < num_blocks ? begin + blocks_per_segment : num_blocks;
        for (int column0 = 0; column0 < rows; column0 += columns_per_pass) {
            const int column = column0 + column_local;
            if (segment < segments && column < rows) {
                int total = 0, before = 0, own = 0;
#pragma unroll 8
                for (int b = begin; b < end; ++b) {
                    const int count = block_counts[static_cast<int64_t>(b) * rows + column];
                    total += count;
                    before += b < block ? count : 0;
                    own = b == block ? count : own;
                }
                if (segments == 1) {
                    column_total[column] = total;
                    slot_base[column] = before;
                } else {
                    atomicAdd(&column_total[column], total);
                    atomicAdd(&slot_base[column], before);
                }
                if (block >= begin && block < end)
                    order_base[column] = own;
            }
        }
        if (block == 0) {
            int bad = 0;
            for (int b = tid; b < num_blocks; b += threads)
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
            slot_base[column] = before;
        }
    }
    __syncthreads();

    const int per_thread = (local_experts + threads - 1) / threads;
    const int first = tid * per_thread < local_experts ? tid * per_thread : local_experts;
    const int last = first + per_thread < local_experts ? first + per_thread : local_experts;
    int64_t padded_sum = 0, count_sum = 0;
    int own_sum = 0, before_sum = 0;
    for (int e = first; e < last; ++e) {
        if (kFusedScan) {
            const int64_t count = column_total[e];
            count_sum += count;
            padded_sum += round_up_to(count, alignment);
        }
        own_sum += order_base[e];
        before_sum += slot_base[e];
    }
    const int64_t padded_scan = kFusedScan ? wave_inclusive_scan(padded_sum) : 0;
    const int64_t assigned_scan = kFusedScan ? wave_inclusive_scan(count_sum) : 0;
    const int own_scan = static_cast<int>(wave_inclusive_scan(own_sum));
    const int before_scan = static_cast<int>(wave_inclusive_scan(before_sum));
    const int wave = tid / kWave;
    const int waves = threads / kWave;
    if ((tid & (kWave - 1)) == kWave - 1) {
        wave_padded[wave] = padded_scan;
        wave_assigned[wave] = assigned_scan;
        wave_own[wave] = own_scan;
        wave_before[wave] = before_scan;
    }
    __syncthreads();
    int64_t running = padded_scan - padded_sum;
    int running_own = own_scan - own_sum;
    int64_t capacity = 0, assigned = 0;
    int own_total = 0, assigned_before = 0;  // this block's assignments, and those of the blocks before it
    for (int w = 0; w < waves; ++w) {
        running += w < wave ? wave_padded[w] : 0;
        running_own += w < wave ? wave_own[w] : 0;
        capacity += wave_padded[w];
        assigned += wave_assigned[w];
        own_total += wave_own[w];
        assigned_before += wave_before[w];
    }
    if (!kFusedScan)
        assigned = totals[0];
    for (int e = first; e < last; ++e) {
        if (kFusedScan) {
            const int64_t count = column_total[e];
            if (block == 0) {
                expert_counts[e] = count;
                expert_offsets[e] = running;
            }
            slot_base[e] += static_cast<int32_t>(running);
            running += round_up_to(count, alignment);
        } else {
            slot_base[e] += static_cast<int32_t>(expert_offsets[e]);
        }
        const int own = order_base[e];
        order_base[e] = running_own;
        running_own += own;
    }
    if (kFusedScan && block == 0 && tid == 0) {
        const int64_t received = column_total[local_experts];
        expert_offsets[local_experts] = capacity;
        send_counts[0] = received;
        recv_rank_prefix[0] = received;
        host_counts[1] = capacity;
        host_counts[2] = assigned;
        host_counts[3] = status_bits;
        __threadfence_system();
        __hip_atomic_store(&host_counts[0], received, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    __syncthreads();
    // The list is dense: this block's run starts where the earlier blocks' assignments end.  Every
    // block also clears as many entries of the unused tail [A, entries) as it has masked choices.
    int64_t* order = nullptr;
    if (slot_order != nullptr) {
        order = slot_order + assigned_before;
        const int64_t block_entries = static_cast<int64_t>(tokens_per_block) * num_topk;
        int64_t* tail = slot_order + assigned + (block * block_entries - assigned_before);
        const int holes = static_cast<int>(block_entries) - own_total;
        for (int i = tid; i < holes; i += threads)
            tail[i] = -1;
        if (block == 0 && tid == 0)
            slot_order[num_blocks * block_entries] = assigned;  // count word behind the list
    }
    if (live)
        assign_token_slots<kCap>(token, num_topk, expand, row_in_block, slot_base[local_experts], slot_base, order_base,
                                 packed_rank, recv_metadata, dst_slots, token_slots, order);
}

template <int kCap, bool kFusedScan>
__global__ void __launch_bounds__(256) layout_assign_kernel(const int32_t* __restrict__ block_counts,
                                                            const int32_t* __restrict__ block_status,
                                                            int num_blocks,
                                                            int64_t num_tokens,
                                                            int num_topk,
                                                            int local_experts,
                                                            int tokens_per_block,
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
                                                            int64_t* slot_order) {
    layout_assign_block<kCap, kFusedScan>(block_counts, block_status, num_blocks, num_tokens, num_topk, local_experts,
                                          tokens_per_block, threads, expand, alignment, packed_rank, local_row, expert_counts,
                                          expert_offsets, send_counts, recv_rank_prefix, totals, host_counts, recv_metadata,
                                          dst_slots, token_slots, slot_order);
}

// Whole layout in one launch when all tokens fit one block: the count pass, then (its results are
// this workgroup's own global writes, made visible by the fence and the barrier) the assignment pass.
template <int kCap>
__global__ void __launch_bounds__(256) layout_single_block_kernel(const int64_t* topk_idx,
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
    layout_count_block<kCap>(topk_idx, num_tokens, num_topk, local_experts, words, threads, snapshot, block_counts,
                             block_status, packed_rank, local_row);
    __threadfence();
    __syncthreads();
    layout_assign_block<kCap, true>(block_counts, block_status, 1, num_tokens, num_topk, local_experts, words * 32, threads,
                                    expand, alignment, packed_rank, local_row, expert_counts, expert_offsets, send_counts,
                                    recv_rank_prefix, nullptr, host_counts, recv_metadata, dst_slots, token_slots, slot_order);
}

// ---------------------------------------------------------------------------------------------
// Dispatch permute / expand
// ---------------------------------------------------------------------------------------------

template <bool kNonTemporal>
__device__ __forceinline__ u32x4 load_vec(const u32x4* p) {
    if constexpr (kNonTemporal)
        return __builtin_nontemporal_load(p);
    else
        return *p;
}

template <bool kNonTemporal>
__device__ __forceinline__ void store_vec(u32x4* p, u32x4 v) {
    if constexpr (kNonTemporal)
        __builtin_nontemporal_store(v, p);
    else
        *p = v;
}

// Load through the scalar data path: the address must be wave-uniform and the memory read-only for
// the duration of the kernel (true of all handle tensors here).  Keeps lookups out of the vector
// memory pipeline and their results in SGPRs.
template <class T>
__device__ __forceinline__ T uniform_load(const T* p) {
    return *(const __attribute__((address_space(4))) T*)(p);
}

// Workgroups are handed to the 8 XCDs round-robin by their linear id, and every XCD has its own L2.
constexpr int kNumXcds = 8;

// n / d for n < 2^31 as one 64-bit multiply and shift: magic = ceil(2^shift / d), shift = 31 + ceil(log2 d).
struct FastDivisor {
    uint32_t magic;
    uint32_t shift;
};

FastDivisor make_fast_divisor(uint32_t divisor) {
    uint32_t log2_ceil = 0;
    while ((uint64_t{1} << log2_ceil) < divisor)
        ++log2_ceil;
    const uint32_t shift = 31 + log2_ceil;
    const uint64_t power = uint64_t{1} << shift;
    return {static_cast<uint32_t>((power + divisor - 1) / divisor), shift};
}

__device__ __forceinline__ uint32_t fast_divide(uint32_t n, uint32_t magic, uint32_t shift) {
    return static_cast<uint32_t>((static_cast<uint64_t>(n) * magic) >> shift);
}

// Kernel arguments are fetched with scalar loads where they are first used, which strings several
// dependent round trips along a short wavefront's life.  Naming them in an empty asm statement at
// the top of the kernel makes the compiler fetch them all in one batch.
#define NANOEP_FETCH_ARGS_2(a, b) asm volatile("" ::"s"(a), "s"(b))
#define NANOEP_FETCH_ARGS_4(a, b, c, d) asm volatile("" ::"s"(a), "s"(b), "s"(c), "s"(d))

// One wavefront moves one 1 KiB chunk (64 lanes x 16 bytes) of one destination row with exactly
// one 128-bit load and one nontemporal 128-bit store per lane: on this part a wavefront that issues
// a single store and retires sustains more HBM write bandwidth than one that issues several.
//
// A workgroup is (64, chunks_per_block, rows_per_block): threadIdx.y is the chunk, threadIdx.z the
// destination candidate, so no per-wave division by the chunk count is needed.  Candidates are
// ordered (source token, k): the K destinations of a token are handled by consecutive workgroups
// behind one XCD's L2, so only the first read of a source row goes to HBM, and every destination
// row is written as one contiguous run by the wavefronts of one workgroup.  The source address
// depends only on the block index, so its load is in flight while the wave-uniform lookups
// (token_slots[t][k], or dst_slots[t] -> recv_metadata[row][2+k] for a handle without that table)
// resolve the destination row.
//
// Zero-fill workgroups clear the alignment gaps: workgroup (e, g) owns gap candidates
// j = g * waves .. of expert e, row offsets[e] + counts[e] + j while that is below offsets[e+1].
// Every XCD takes one contiguous range of the copy work followed by one contiguous range of the
// zero-fill work, so it gets its share of both.

// How a token-order dispatch wavefront finds its destination row.
enum DispatchLookup {
    kLookupMetadata = 0,  // dst_slots -> recv_metadata row -> field k
    kLookupTable = 1,     // token_slots[token][k]
};

// One zero-fill workgroup: each wavefront clears one whole gap row (and its weight).
__device__ __forceinline__ void zero_fill_gap_rows(uint32_t block,
                                                   uint32_t pad_per_expert,
                                                   uint32_t pad_groups_per_expert,
                                                   uint32_t chunks_per_block,
                                                   uint32_t rows_per_block,
                                                   const int64_t* __restrict__ expert_counts,
                                                   const int64_t* __restrict__ expert_offsets,
                                                   u32x4* __restrict__ recv_x,
                                                   float* __restrict__ recv_weights,
                                                   int64_t out_rows,
                                                   int vectors) {
    const uint32_t wave_y = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const uint32_t wave_z = __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t expert = block / pad_groups_per_expert;
    const uint32_t group = block - expert * pad_groups_per_expert;
    const uint32_t waves = chunks_per_block * rows_per_block;
    const uint32_t j = group * waves + wave_z * chunks_per_block + wave_y;
    if (j >= pad_per_expert)
        return;
    const int64_t out_row = uniform_load(expert_offsets + expert) + uniform_load(expert_counts + expert) + j;
    if (out_row >= uniform_load(expert_offsets + expert + 1) || out_row >= out_rows)
        return;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    u32x4* dst = recv_x + out_row * vectors;
    for (int vector = threadIdx.x; vector < vectors; vector += kWave)
        store_vec<true>(dst + vector, zero);
    if (threadIdx.x == 0 && recv_weights != nullptr)
        recv_weights[out_row] = 0.0f;
}

template <int kLookup, bool kZeroFill>
__global__ void __launch_bounds__(1024) dispatch_rows_kernel(const u32x4* __restrict__ x,                // [T][vectors]
                                                             const float* __restrict__ weights,         // [T][K] or null
                                                             const int32_t* __restrict__ recv_metadata,  // [N][K+2]
                                                             const int64_t* __restrict__ dst_slots,     // [T]
                                                             const int32_t* __restrict__ token_slots,   // [T][K] or null
                                                             const int64_t* __restrict__ expert_counts,
                                                             const int64_t* __restrict__ expert_offsets,
                                                             u32x4* __restrict__ recv_x,                // [C or N][vectors]
                                                             int64_t* __restrict__ recv_topk_idx,       // compact [N][K] or null
                                                             float* __restrict__ recv_weights,          // [C] / [N][K] or null
                                                             int64_t recv_count,
                                                             int64_t out_rows,
                                                             uint32_t copy_candidates,  // T*K expanded, T compact
                                                             uint32_t copy_blocks,
                                                             uint32_t copy_per_xcd,  // ceil(copy_blocks / 8)
                                                             uint32_t pad_blocks,
                                                             uint32_t pad_per_xcd,   // ceil(pad_blocks / 8)
                                                             uint32_t parts,            // workgroups per candidate group (rows longer than 16 chunks)
                                                             uint32_t parts_magic,      // fast divisor by parts
                                                             uint32_t parts_shift,
                                                             uint32_t chunks_per_block,  // == blockDim.y
                                                             uint32_t rows_per_block,    // == blockDim.z
                                                             uint32_t pad_per_expert,
                                                             uint32_t pad_groups_per_expert,
                                                             int vectors,
                                                             int chunks,
                                                             int num_topk,
                                                             int topk_shift,  // log2(K) when K is a power of two, else -1
                                                             int expand) {
    NANOEP_FETCH_ARGS_4(x, weights, recv_x, recv_weights);
    NANOEP_FETCH_ARGS_4(token_slots, copy_blocks, dst_slots, recv_metadata);
    NANOEP_FETCH_ARGS_4(out_rows, recv_count, copy_candidates, copy_per_xcd);
    NANOEP_FETCH_ARGS_4(parts_magic, parts_shift, vectors, chunks);
    NANOEP_FETCH_ARGS_4(num_topk, topk_shift, expand, chunks_per_block);
    // Workgroups are handed to the XCDs round-robin.  Each XCD takes one contiguous range of the
    // copy work followed by one contiguous range of the zero-fill work, so neighbouring work items
    // (which share their source rows) stay behind one L2 and every XCD gets its share of both.
    // (kZeroFill is false when the launch has no zero-fill work: the copy path then carries none of
    // its bookkeeping, which shows in a wavefront that lives about a microsecond)
    const uint32_t xcd = blockIdx.x % kNumXcds;
    const uint32_t index_in_xcd = blockIdx.x / kNumXcds;
    const bool copy_work = !kZeroFill || index_in_xcd < copy_per_xcd;
    uint32_t block = xcd * copy_per_xcd + index_in_xcd;
    if (kZeroFill && !copy_work)
        block = xcd * pad_per_xcd + (index_in_xcd - copy_per_xcd);
    if (copy_work ? (index_in_xcd >= copy_per_xcd || block >= copy_blocks)
                  : (index_in_xcd - copy_per_xcd >= pad_per_xcd || block >= pad_blocks))
        return;
    const int lane = threadIdx.x;
    const uint32_t wave_y = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const uint32_t wave_z = __builtin_amdgcn_readfirstlane(threadIdx.z);

    if (copy_work) {
        const uint32_t group = fast_divide(block, parts_magic, parts_shift);
        const uint32_t part = block - group * parts;
        const uint32_t candidate = group * rows_per_block + wave_z;
        const int chunk = static_cast<int>(part * chunks_per_block + wave_y);
        if (candidate >= copy_candidates || chunk >= chunks)
            return;
        const int vector = chunk * kWave + lane;
        const bool in_row = vector < vectors;
        uint32_t token = candidate;
        int k = 0;
        int64_t out_row;
        const int32_t* fields = nullptr;
        if (expand) {
            token = topk_shift >= 0 ? candidate >> topk_shift : candidate / static_cast<uint32_t>(num_topk);
            k = static_cast<int>(candidate - token * num_topk);
        }
        token = __builtin_amdgcn_readfirstlane(token);
        k = __builtin_amdgcn_readfirstlane(k);
        // lanes past the end of a short row re-read vector 0 instead of branching around the load
        const u32x4 data = x[static_cast<int64_t>(token) * vectors + (in_row ? vector : 0)];
        if (kLookup == kLookupTable && expand) {
            out_row = uniform_load(token_slots + static_cast<int64_t>(token) * num_topk + k);
        } else {
            const int64_t row = uniform_load(dst_slots + token);
            if (row < 0 || row >= recv_count)
                return;
            fields = recv_metadata + row * (num_topk + 2);
            out_row = expand ? static_cast<int64_t>(uniform_load(fields + 2 + k)) : row;
        }
        if (out_row < 0 || out_row >= out_rows)
            return;
        if (in_row)
            store_vec<true>(recv_x + out_row * vectors + vector, data);
        if (chunk != 0)
            return;
        if (expand) {
            if (lane == 0 && recv_weights != nullptr)
                recv_weights[out_row] = weights[static_cast<int64_t>(token) * num_topk + k];
        } else if (lane < num_topk) {
            if (recv_topk_idx != nullptr)
                recv_topk_idx[out_row * num_topk + lane] = fields[2 + lane];
            if (recv_weights != nullptr)
                recv_weights[out_row * num_topk + lane] = weights[static_cast<int64_t>(token) * num_topk + lane];
        }
    } else {
        zero_fill_gap_rows(block, pad_per_expert, pad_groups_per_expert, chunks_per_block, rows_per_block, expert_counts,
                           expert_offsets, recv_x, recv_weights, out_rows, vectors);
    }
}

// The slot-order walk, stripped to what its wavefronts need: a wavefront lives about a microsecond,
// most of it waiting in a chain of scalar work -> list entry -> source load -> store, so every
// scalar instruction and branch ahead of the source load is throughput.  Validity is folded into
// one flag and the load is issued unconditionally (row 0 stands in).  kZeroFill is false when the
// launch has no gap rows to clear: the copy path then carries none of that bookkeeping.
template <bool kDeviceCount, bool kZeroFill>
__global__ void __launch_bounds__(1024) dispatch_ordered_kernel(const u32x4* __restrict__ x,              // [T][vectors]
                                                                const float* __restrict__ weights,       // [T][K] or null
                                                                const int64_t* __restrict__ slot_order,  // [entries]
                                                                const int64_t* __restrict__ live_count,  // device entry count (kDeviceCount)
                                                                const int64_t* __restrict__ expert_counts,
                                                                const int64_t* __restrict__ expert_offsets,
                                                                u32x4* __restrict__ recv_x,        // [C][vectors]
                                                                float* __restrict__ recv_weights,  // [C] or null
                                                                uint32_t entries,
                                                                uint32_t source_limit,  // T*K
                                                                uint32_t out_rows,
                                                                uint32_t copy_blocks,
                                                                uint32_t copy_per_xcd,
                                                                uint32_t pad_blocks,
                                                                uint32_t pad_per_xcd,
                                                                uint32_t pad_per_expert,
                                                                uint32_t pad_groups_per_expert,
                                                                uint32_t parts,
                                                                uint32_t parts_magic,
                                                                uint32_t parts_shift,
                                                                uint32_t chunks_per_block,  // == blockDim.y
                                                                uint32_t rows_per_block,    // == blockDim.z
                                                                uint32_t vectors,
                                                                uint32_t chunks,
                                                                uint32_t topk_magic,  // fast divisor by K
                                                                uint32_t topk_shift) {
    NANOEP_FETCH_ARGS_4(x, weights, recv_x, recv_weights);
    NANOEP_FETCH_ARGS_4(slot_order, entries, source_limit, out_rows);
    NANOEP_FETCH_ARGS_4(copy_blocks, copy_per_xcd, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    NANOEP_FETCH_ARGS_4(chunks, topk_magic, topk_shift, live_count);
    if (kDeviceCount) {
        // The list length was not known when the grid was sized: shrink the walk to the entries in
        // use, so that the per-XCD ranges split the real work and not its unused tail.
        const int64_t live = uniform_load(live_count);
        if (live >= 0 && live < static_cast<int64_t>(entries)) {
            entries = static_cast<uint32_t>(live);
            copy_blocks = (rows_per_block == 1 ? entries : (entries + rows_per_block - 1) / rows_per_block) * parts;
            copy_per_xcd = (copy_blocks + kNumXcds - 1) / kNumXcds;
        }
    }
    const uint32_t index_in_xcd = blockIdx.x / kNumXcds;
    if (kZeroFill && index_in_xcd >= copy_per_xcd) {
        const uint32_t pad_index = index_in_xcd - copy_per_xcd;
        const uint32_t pad_block = (blockIdx.x % kNumXcds) * pad_per_xcd + pad_index;
        if (pad_index < pad_per_xcd && pad_block < pad_blocks)
            zero_fill_gap_rows(pad_block, pad_per_expert, pad_groups_per_expert, chunks_per_block, rows_per_block,
                               expert_counts, expert_offsets, recv_x, recv_weights, out_rows, static_cast<int>(vectors));
        return;
    }
    const uint32_t block = (blockIdx.x % kNumXcds) * copy_per_xcd + index_in_xcd;
    if (index_in_xcd >= copy_per_xcd || block >= copy_blocks)
        return;
    const uint32_t group = fast_divide(block, parts_magic, parts_shift);
    const uint32_t part = block - group * parts;
    const uint32_t candidate = group * rows_per_block + __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t chunk = part * chunks_per_block + __builtin_amdgcn_readfirstlane(threadIdx.y);
    if (candidate >= entries || chunk >= chunks)
        return;
    const int64_t entry = uniform_load(slot_order + candidate);
    const uint32_t source = static_cast<uint32_t>(entry);
    const uint32_t out_row = static_cast<uint32_t>(static_cast<uint64_t>(entry) >> 32);
    const bool valid = entry >= 0 && source < source_limit && out_row < out_rows;
    const uint32_t token = valid ? fast_divide(source, topk_magic, topk_shift) : 0u;
    const uint32_t vector = chunk * kWave + threadIdx.x;
    const bool in_row = vector < vectors;
    const u32x4 data = x[static_cast<uint64_t>(token) * vectors + (in_row ? vector : 0u)];
    if (!valid)
        return;
    if (in_row)
        store_vec<true>(recv_x + static_cast<uint64_t>(out_row) * vectors + vector, data);
    if (chunk == 0 && threadIdx.x == 0 && recv_weights != nullptr)
        recv_weights[out_row] = weights[source];
}

// Compact layout: receive row r holds source token src_token(r), in token order, so the dispatch is
// a row copy with holes.  Nothing is re-used, so workgroups walk the rows in plain launch order
// (one linear stream over the whole device) and the kernel carries nothing but the copy.
__global__ void __launch_bounds__(1024) dispatch_compact_kernel(const u32x4* __restrict__ x,                // [T][vectors]
                                                                const float* __restrict__ weights,         // [T][K] or null
                                                                const int32_t* __restrict__ recv_metadata,  // [N][K+2]
                                                                const int64_t* __restrict__ dst_slots,     // [T]
                                                                u32x4* __restrict__ recv_x,                // [N][vectors]
                                                                int64_t* __restrict__ recv_topk_idx,       // [N][K] or null
                                                                float* __restrict__ recv_weights,          // [N][K] or null
                                                                uint32_t tokens,
                                                                uint32_t recv_count,
                                                                uint32_t parts,
                                                                uint32_t parts_magic,
                                                                uint32_t parts_shift,
                                                                uint32_t chunks_per_block,  // == blockDim.y
                                                                uint32_t rows_per_block,    // == blockDim.z
                                                                uint32_t vectors,
                                                                uint32_t chunks,
                                                                uint32_t topk) {
    NANOEP_FETCH_ARGS_4(x, dst_slots, recv_x, tokens);
    NANOEP_FETCH_ARGS_4(recv_count, parts, parts_magic, parts_shift);
    NANOEP_FETCH_ARGS_4(chunks_per_block, rows_per_block, vectors, chunks);
    const uint32_t group = fast_divide(blockIdx.x, parts_magic, parts_shift);
    const uint32_t part = blockIdx.x - group * parts;
    const uint32_t token = group * rows_per_block + __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t chunk = part * chunks_per_block + __builtin_amdgcn_readfirstlane(threadIdx.y);
    if (token >= tokens || chunk >= chunks)
        return;
    const uint32_t vector = chunk * kWave + threadIdx.x;
    const bool in_row = vector < vectors;
    // the source address depends on the block index alone: its load is in flight during the lookup
    const u32x4 data = x[static_cast<uint64_t>(token) * vectors + (in_row ? vector : 0u)];
    const int64_t row = uniform_load(dst_slots + token);
    if (row < 0 || row >= static_cast<int64_t>(recv_count))
        return;
    if (in_row)
        store_vec<true>(recv_x + static_cast<uint64_t>(row) * vectors + vector, data);
    if (chunk == 0 && threadIdx.x < topk) {
        const uint32_t lane = threadIdx.x;
        if (recv_topk_idx != nullptr)
            recv_topk_idx[row * topk + lane] = recv_metadata[row * (topk + 2) + 2 + lane];
        if (recv_weights != nullptr)
            recv_weights[row * topk + lane] = weights[static_cast<uint64_t>(token) * topk + lane];
    }
}

// ---------------------------------------------------------------------------------------------
// Combine gather-reduce
// ---------------------------------------------------------------------------------------------

__device__ __forceinline__ float bf16_low(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_high(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Round to nearest even; NaN becomes the canonical quiet NaN.
__device__ __forceinline__ uint32_t bf16_round(float value) {
    uint32_t bits = __float_as_uint(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u)
        return 0x7fc0u;
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return bits >> 16;
}

__device__ __forceinline__ void accumulate(float (&acc)[8], const u32x4 v) {
    acc[0] += bf16_low(v.x);
    acc[1] += bf16_high(v.x);
    acc[2] += bf16_low(v.y);
    acc[3] += bf16_high(v.y);
    acc[4] += bf16_low(v.z);
    acc[5] += bf16_high(v.z);
    acc[6] += bf16_low(v.w);
    acc[7] += bf16_high(v.w);
}

// One wavefront produces one 1 KiB chunk of one source token's output row.  A workgroup is
// (64, chunks_per_block, tokens_per_block).  Lane k fetches the token's k-th slot (from
// token_slots[t][k], or dst_slots[t] -> recv_metadata[row][2+k]); the slots are broadcast to
// scalars, the kGroup rows are fetched with back-to-back nontemporal 128-bit loads (a masked k
// re-reads row 0 so that the loads stay unconditional) and the valid ones are added in ascending k
// starting from +0.0f; the optional bias is added once and the sum is rounded to bf16 once.
template <int kGroup, bool kDirectSlots>
__global__ void __launch_bounds__(1024) combine_rows_kernel(const u32x4* __restrict__ y,                // [rows][vectors]
                                                            const float* __restrict__ weights,         // [C] / [N][K] or null
                                                            const u32x4* __restrict__ bias,            // [T][vectors] or null
                                                            const int32_t* __restrict__ recv_metadata,  // [N][K+2]
                                                            const int64_t* __restrict__ dst_slots,     // [T]
                                                            const int32_t* __restrict__ token_slots,   // [T][K] or null
                                                            u32x4* __restrict__ out_x,                 // [T][vectors]
                                                            float* __restrict__ out_weights,           // [T][K] or null
                                                            int64_t recv_count,
                                                            int64_t y_rows,
                                                            uint32_t num_tokens,
                                                            uint32_t parts,
                                                            uint32_t parts_magic,  // fast divisor by parts
                                                            uint32_t parts_shift,
                                                            uint32_t chunks_per_block,  // == blockDim.y
                                                            uint32_t tokens_per_block,  // == blockDim.z
                                                            int vectors,
                                                            int chunks,
                                                            int num_topk,
                                                            int expand,
                                                            int multiple_reduction) {
    NANOEP_FETCH_ARGS_4(y, weights, bias, out_x);
    NANOEP_FETCH_ARGS_4(recv_metadata, dst_slots, token_slots, out_weights);
    NANOEP_FETCH_ARGS_4(recv_count, y_rows, num_tokens, parts);
    NANOEP_FETCH_ARGS_4(parts_magic, parts_shift, chunks_per_block, tokens_per_block);
    NANOEP_FETCH_ARGS_4(vectors, chunks, num_topk, expand);
    const int lane = threadIdx.x;
    const uint32_t wave_y = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const uint32_t wave_z = __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t group = fast_divide(blockIdx.x, parts_magic, parts_shift);
    const uint32_t part = blockIdx.x - group * parts;
    const uint32_t token = __builtin_amdgcn_readfirstlane(group * tokens_per_block + wave_z);
    const int chunk = static_cast<int>(part * chunks_per_block + wave_y);
    if (token >= num_tokens || chunk >= chunks)
        return;
    const int vector = chunk * kWave + lane;
    const bool in_row = vector < vectors;
    // lanes past the end of a short row re-read vector 0 instead of branching around the loads
    const int load_vector = in_row ? vector : 0;

    // field: expanded slot (or local expert id when compact) of this token's k = lane, -1 when masked
    int64_t row = -1;
    bool received = true;
    const int32_t* fields;
    if (kDirectSlots) {
        fields = token_slots + static_cast<int64_t>(token) * num_topk;
    } else {
        row = uniform_load(dst_slots + token);
        received = row >= 0 && row < recv_count;
        fields = recv_metadata + (received ? row : 0) * (num_topk + 2) + 2;
    }
    // Compact rows need their per-k fields only to return weights: a received row always carries
    // at least one valid choice, so the payload path skips that dependent load.
    const bool need_fields = expand || (chunk == 0 && out_weights != nullptr);
    int field = -1;
    if (need_fields && received && lane < num_topk)
        field = fields[lane];
    const bool valid = expand ? (field >= 0 && field < y_rows) : field >= 0;
    const uint64_t valid_mask = __ballot(valid);
    // compact: the token's single received row stands in for k = 0
    const uint64_t gather_mask = expand ? valid_mask : ((received && row < y_rows) ? 1ull : 0ull);
    const int gathered = gather_mask == 0 ? 0 : (expand ? num_topk : 1);

    u32x4 bias_data = {0u, 0u, 0u, 0u};
    if (bias != nullptr)
        bias_data = load_vec<true>(bias + static_cast<int64_t>(token) * vectors + load_vector);

    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int base = 0; base < gathered; base += kGroup) {
        u32x4 data[kGroup];
#pragma unroll
        for (int k = 0; k < kGroup; ++k) {
            const bool live = (gather_mask >> (base + k)) & 1;
            int64_t source_row = 0;
            if (live)
                source_row = expand ? static_cast<int64_t>(__builtin_amdgcn_readlane(field, (base + k) & (kWave - 1))) : row;
            data[k] = load_vec<true>(y + source_row * vectors + load_vector);
        }
#pragma unroll
        for (int k = 0; k < kGroup; ++k)
            if ((gather_mask >> (base + k)) & 1)
                accumulate(acc, data[k]);
    }
    if (multiple_reduction && expand && __popcll(valid_mask) >= 2) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            acc[j] = 0.0f + __uint_as_float(bf16_round(acc[j]) << 16);
    }
    if (bias != nullptr)
        accumulate(acc, bias_data);
    if (in_row) {
        u32x4 packed;
        packed.x = bf16_round(acc[0]) | (bf16_round(acc[1]) << 16);
        packed.y = bf16_round(acc[2]) | (bf16_round(acc[3]) << 16);
        packed.z = bf16_round(acc[4]) | (bf16_round(acc[5]) << 16);
        packed.w = bf16_round(acc[6]) | (bf16_round(acc[7]) << 16);
        store_vec<true>(out_x + static_cast<int64_t>(token) * vectors + vector, packed);
    }

    if (chunk == 0 && out_weights != nullptr && lane < num_topk) {
        float weight = 0.0f;
        if (valid)
            weight = expand ? weights[field] : weights[row * num_topk + lane];
        out_weights[static_cast<int64_t>(token) * num_topk + lane] = weight;
    }
}

__global__ void __launch_bounds__(kBlockThreads) copy_vectors_kernel(const u32x4* __restrict__ src,
                                                                    u32x4* __restrict__ dst,
                                                                    size_t vectors) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < vectors)
        dst[i] = src[i];
}

// ---------------------------------------------------------------------------------------------
// Launch helpers
// ---------------------------------------------------------------------------------------------

// Expanded layout with at most kTopk <= 4 rows per token and the slot table at hand: the same
// gather-sum as combine_rows_kernel, carrying only what that case needs (the token's slots come as
// scalars straight from the table).  With so few rows per token the kernel is short and close to a
// copy, and the general kernel's bookkeeping showed (Mixtral-shaped batch: 19.3 us against 17.3 us
// for the bare access pattern).
template <int kTopk>
__global__ void __launch_bounds__(1024) combine_few_rows_kernel(const u32x4* __restrict__ y,              // [C][vectors]
                                                                const float* __restrict__ weights,       // [C] or null
                                                                const u32x4* __restrict__ bias,          // [T][vectors] or null
                                                                const int32_t* __restrict__ token_slots,  // [T][K]
                                                                u32x4* __restrict__ out_x,               // [T][vectors]
                                                                float* __restrict__ out_weights,         // [T][K] or null
                                                                uint32_t tokens,
                                                                uint32_t y_rows,
                                                                uint32_t parts,
                                                                uint32_t parts_magic,
                                                                uint32_t parts_shift,
                                                                uint32_t chunks_per_block,  // == blockDim.y
                                                                uint32_t rows_per_block,    // == blockDim.z
                                                                uint32_t vectors,
                                                                uint32_t chunks,
                                                                uint32_t topk,
                                                                int multiple_reduction) {
    NANOEP_FETCH_ARGS_4(y, token_slots, out_x, bias);
    NANOEP_FETCH_ARGS_4(tokens, y_rows, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    NANOEP_FETCH_ARGS_4(chunks, topk, multiple_reduction, out_weights);
    const uint32_t group = fast_divide(blockIdx.x, parts_magic, parts_shift);
    const uint32_t part = blockIdx.x - group * parts;
    const uint32_t token = group * rows_per_block + __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t chunk = part * chunks_per_block + __builtin_amdgcn_readfirstlane(threadIdx.y);
    if (token >= tokens || chunk >= chunks)
        return;
    const uint32_t vector = chunk * kWave + threadIdx.x;
    const bool in_row = vector < vectors;
    const uint32_t load_vector = in_row ? vector : 0u;
    const int32_t* slots = token_slots + static_cast<uint64_t>(token) * topk;
    int32_t slot[kTopk];
    bool valid[kTopk];
#pragma unroll
    for (int k = 0; k < kTopk; ++k) {
        slot[k] = uniform_load(slots + (static_cast<uint32_t>(k) < topk ? k : 0));
        valid[k] = static_cast<uint32_t>(k) < topk && slot[k] >= 0 && static_cast<uint32_t>(slot[k]) < y_rows;
    }
    u32x4 data[kTopk];
#pragma unroll
    for (int k = 0; k < kTopk; ++k)  // a masked k re-reads row 0 and drops it: the loads stay unconditional
        data[k] = load_vec<true>(y + static_cast<uint64_t>(valid[k] ? slot[k] : 0) * vectors + load_vector);
    u32x4 bias_data = {0u, 0u, 0u, 0u};
    if (bias != nullptr)
        bias_data = load_vec<true>(bias + static_cast<uint64_t>(token) * vectors + load_vector);
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    int valid_count = 0;
#pragma unroll
    for (int k = 0; k < kTopk; ++k) {
        if (valid[k]) {
            accumulate(acc, data[k]);
            ++valid_count;
        }
    }
    if (multiple_reduction && valid_count >= 2) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            acc[j] = 0.0f + __uint_as_float(bf16_round(acc[j]) << 16);
    }
    if (bias != nullptr)
        accumulate(acc, bias_data);
    if (in_row) {
        u32x4 packed;
        packed.x = bf16_round(acc[0]) | (bf16_round(acc[1]) << 16);
        packed.y = bf16_round(acc[2]) | (bf16_round(acc[3]) << 16);
        packed.z = bf16_round(acc[4]) | (bf16_round(acc[5]) << 16);
        packed.w = bf16_round(acc[6]) | (bf16_round(acc[7]) << 16);
        store_vec<true>(out_x + static_cast<uint64_t>(token) * vectors + vector, packed);
    }
    if (chunk == 0 && out_weights != nullptr && threadIdx.x < topk) {
        const int32_t mine = slots[threadIdx.x];
        const bool mine_valid = mine >= 0 && static_cast<uint32_t>(mine) < y_rows;
        out_weights[static_cast<uint64_t>(token) * topk + threadIdx.x] = mine_valid ? weights[mine] : 0.0f;
    }
}

// Compact layout: a token has one received row, so the combine is a row copy through fp32
// (0.0f + x, which turns -0 into +0 and quiets NaNs, then the bias) with holes: tokens that were
// not sent get 0 (+bias).  Plain launch order, nothing but the copy in the kernel.
__global__ void __launch_bounds__(1024) combine_compact_kernel(const u32x4* __restrict__ y,                // [N][vectors]
                                                               const float* __restrict__ weights,         // [N][K] or null
                                                               const u32x4* __restrict__ bias,            // [T][vectors] or null
                                                               const int32_t* __restrict__ recv_metadata,  // [N][K+2]
                                                               const int64_t* __restrict__ dst_slots,     // [T]
                                                               u32x4* __restrict__ out_x,                 // [T][vectors]
                                                               float* __restrict__ out_weights,           // [T][K] or null
                                                               uint32_t tokens,
                                                               uint32_t recv_count,
                                                               uint32_t parts,
                                                               uint32_t parts_magic,
                                                               uint32_t parts_shift,
                                                               uint32_t chunks_per_block,  // == blockDim.y
                                                               uint32_t rows_per_block,    // == blockDim.z
                                                               uint32_t vectors,
                                                               uint32_t chunks,
                                                               uint32_t topk) {
    NANOEP_FETCH_ARGS_4(y, dst_slots, out_x, bias);
    NANOEP_FETCH_ARGS_4(tokens, recv_count, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    const uint32_t group = fast_divide(blockIdx.x, parts_magic, parts_shift);
    const uint32_t part = blockIdx.x - group * parts;
    const uint32_t token = group * rows_per_block + __builtin_amdgcn_readfirstlane(threadIdx.z);
    const uint32_t chunk = part * chunks_per_block + __builtin_amdgcn_readfirstlane(threadIdx.y);
    if (token >= tokens || chunk >= chunks)
        return;
    const uint32_t vector = chunk * kWave + threadIdx.x;
    const bool in_row = vector < vectors;
    const uint32_t load_vector = in_row ? vector : 0u;
    const int64_t row = uniform_load(dst_slots + token);
    const bool received = row >= 0 && row < static_cast<int64_t>(recv_count);
    // a token that was not sent re-reads row 0 and drops it: the load stays unconditional
    const u32x4 data = load_vec<true>(y + static_cast<uint64_t>(received ? row : 0) * vectors + load_vector);
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (received)
        accumulate(acc, data);
    if (bias != nullptr)
        accumulate(acc, load_vec<true>(bias + static_cast<uint64_t>(token) * vectors + load_vector));
    if (in_row) {
        u32x4 packed;
        packed.x = bf16_round(acc[0]) | (bf16_round(acc[1]) << 16);
        packed.y = bf16_round(acc[2]) | (bf16_round(acc[3]) << 16);
        packed.z = bf16_round(acc[4]) | (bf16_round(acc[5]) << 16);
        packed.w = bf16_round(acc[6]) | (bf16_round(acc[7]) << 16);
        store_vec<true>(out_x + static_cast<uint64_t>(token) * vectors + vector, packed);
    }
    if (chunk == 0 && out_weights != nullptr && threadIdx.x < topk) {
        const uint32_t lane = threadIdx.x;
        float weight = 0.0f;
        if (received && recv_metadata[row * (topk + 2) + 2 + lane] >= 0)
            weight = weights[row * topk + lane];
        out_weights[static_cast<uint64_t>(token) * topk + lane] = weight;
    }
}

constexpr int kMaxWavesPerBlock = 16;
constexpr int kDefaultChunksPerBlock = 2;

// Workgroup shape (64, chunks_per_block, rows_per_block) for rows of `chunks` 1 KiB chunks; a row
// longer than chunks_per_block is covered by `parts` consecutive workgroups, and rows of a single
// chunk are grouped so that a workgroup still has a few wavefronts.
struct RowBlocking {
    unsigned chunks_per_block;
    unsigned rows_per_block;
    unsigned parts;
};

enum WalkShape {
    kTokenOrderWalk,  // two-wavefront workgroups: best or within noise of best for the expanded token-order walks
    kSlotOrderWalk,   // the row split evenly over workgroups of up to 8 wavefronts
    kRowCopyWalk,     // compact layouts (plain row copies): single-wavefront workgroups
};

RowBlocking pick_row_blocking(int chunks, WalkShape shape) {
    RowBlocking blocking{};
    int per_block = env_int("NANOEP_CHUNKS_PER_BLOCK", 0);
    if (per_block < 1 || per_block > kMaxWavesPerBlock) {
        per_block = kDefaultChunksPerBlock;
        if (shape == kSlotOrderWalk) {
            const int pieces = (chunks + 7) / 8;
            per_block = (chunks + pieces - 1) / pieces;
        } else if (shape == kRowCopyWalk) {
            per_block = 1;
        }
    }
    if (per_block > chunks)
        per_block = chunks;
    blocking.chunks_per_block = static_cast<unsigned>(per_block);
    blocking.parts = static_cast<unsigned>((chunks + per_block - 1) / per_block);
    int rows = 1;
    if (blocking.parts == 1) {
        rows = env_int("NANOEP_ROWS_PER_BLOCK", 0);
        if (rows < 1 || rows * per_block > kMaxWavesPerBlock)
            rows = per_block >= 4 ? 1 : 4 / per_block;
    }
    blocking.rows_per_block = static_cast<unsigned>(rows);
    return blocking;
}

int validate_cu_budget(int num_cus) {
    int device = 0;
    NANOEP_HIP_TRY(hipGetDevice(&device));
    static thread_local int cached_device = -1;
    static thread_local int cached_cus = 0;
    if (device != cached_device) {
        int cus = 0;
        NANOEP_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
        cached_device = device;
        cached_cus = cus;
    }
    return (num_cus < 0 || num_cus > cached_cus) ? NANOEP_ERR_INVALID_ARGUMENT : NANOEP_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace


// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------

extern "C" {

int nanoep_abi_version(void) { return 2; }

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

size_t nanoep_layout_workspace_bytes(int64_t num_tokens, int num_topk, int64_t num_local_experts) {
    if (num_tokens < 0 || num_topk <= 0 || num_local_experts <= 0)
        return 0;
    return carve_layout_workspace(nullptr, num_tokens, num_topk, num_local_experts).bytes;
}

int nanoep_layout_block_tokens(int64_t num_local_experts) {
    return num_local_experts <= 0 ? 0 : layout_tokens_per_block(num_local_experts);
}

int64_t nanoep_slot_order_entries(int64_t num_tokens, int num_topk, int64_t num_local_experts) {
    if (num_tokens < 0 || num_topk <= 0 || num_local_experts <= 0)
        return 0;
    const int per_block = layout_tokens_per_block(num_local_experts);
    if (per_block == 0 || num_tokens == 0)
        return 0;
    return (num_tokens + per_block - 1) / per_block * per_block * num_topk + 1;
}

int nanoep_layout(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts,
                  int64_t alignment, int expand, int32_t* recv_metadata, int64_t* expert_counts,
                  int64_t* expert_offsets, int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot,
                  int64_t* recv_rank_prefix, int32_t* token_slots, int64_t* slot_order, void* workspace,
                  size_t workspace_bytes, int64_t* host_counts, void* stream_handle) {
    if (num_tokens < 0 || num_tokens > INT32_MAX || num_topk <= 0 || num_topk > kMaxTopk || num_local_experts <= 0 ||
        num_local_experts >= (int64_t{1} << (31 - kRankBits)) || alignment <= 0 || alignment > (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (expert_counts == nullptr || expert_offsets == nullptr || send_counts == nullptr || recv_rank_prefix == nullptr ||
        host_counts == nullptr || workspace == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (num_tokens > 0 && (topk_idx == nullptr || recv_metadata == nullptr || dst_slots == nullptr || topk_snapshot == nullptr))
        return NANOEP_ERR_INVALID_ARGUMENT;
    // the slot-order list packs token * K + k into 32 bits and only exists for the expanded layout
    if (slot_order != nullptr && (!expand || num_tokens * num_topk >= (int64_t{1} << 31)))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const int tokens_per_block = layout_tokens_per_block(num_local_experts);
    if (tokens_per_block == 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const LayoutWorkspace ws = carve_layout_workspace(workspace, num_tokens, num_topk, num_local_experts);
    if (ws.bytes > workspace_bytes)
        return NANOEP_ERR_WORKSPACE;
    const int64_t blocks64 = (num_tokens + tokens_per_block - 1) / tokens_per_block;
    const int blocks = static_cast<int>(blocks64);
    const int experts = static_cast<int>(num_local_experts);
    const int words = tokens_per_block / 32;
    auto stream = static_cast<hipStream_t>(stream_handle);

    __atomic_store_n(&host_counts[0], int64_t{-1}, __ATOMIC_RELEASE);
    const int count_threads = tokens_per_block < kWave ? kWave : tokens_per_block;
    // Two launches when every block can afford to sum the block histograms itself
    // (blocks x (L+1) loads spread over the workgroup), three with a single-workgroup scan otherwise.
    bool fused_scan = blocks > 0 && static_cast<int64_t>(blocks) * (experts + 1) <= int64_t{32} * count_threads;
    const int forced_launches = env_int("NANOEP_LAYOUT_LAUNCHES", 0);
    if (forced_launches == 3)
        fused_scan = false;
    else if (forced_launches == 2 && blocks > 0)
        fused_scan = true;
    hipError_t launch_status = hipSuccess;
    with_topk_cap(num_topk, [&](auto cap) {
        constexpr int kCap = decltype(cap)::value;
        if (blocks == 1 && forced_launches == 0) {
            const size_t count_lds = static_cast<size_t>(experts + 1) * (words * 6 + 4);
            const size_t assign_lds = static_cast<size_t>(experts + 1) * 12;
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
        const size_t assign_lds = static_cast<size_t>(experts + 1) * 12;
        if (fused_scan) {
            layout_assign_kernel<kCap, true><<<blocks, count_threads, assign_lds, stream>>>(
                ws.block_counts, ws.block_status, blocks, num_tokens, num_topk, experts, tokens_per_block, count_threads,
                expand, alignment, ws.packed_rank, ws.local_row, expert_counts, expert_offsets, send_counts,
                recv_rank_prefix, ws.totals, host_counts, recv_metadata, dst_slots, token_slots, slot_order);
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
                ws.block_counts, ws.block_status, blocks, num_tokens, num_topk, experts, tokens_per_block, count_threads,
                expand, alignment, ws.packed_rank, ws.local_row, expert_counts, expert_offsets, send_counts,
                recv_rank_prefix, ws.totals, host_counts, recv_metadata, dst_slots, token_slots, slot_order);
            launch_status = hipGetLastError();
        }
    });
    NANOEP_HIP_TRY(launch_status);
    return NANOEP_OK;
}

int nanoep_wait_counts(int64_t* host_counts, void* stream_handle, double timeout_seconds,
                       int64_t out[NANOEP_HOST_COUNT_WORDS]) {
    if (host_counts == nullptr || out == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    auto stream = static_cast<hipStream_t>(stream_handle);
    timespec start{};
    clock_gettime(CLOCK_MONOTONIC, &start);
    uint64_t spins = 0;
    while (true) {
        const int64_t received = __atomic_load_n(&host_counts[0], __ATOMIC_ACQUIRE);
        if (received >= 0)
            break;
        if ((++spins & 0x3ff) == 0) {
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
            timespec now{};
            clock_gettime(CLOCK_MONOTONIC, &now);
            const double elapsed = (now.tv_sec - start.tv_sec) + 1e-9 * (now.tv_nsec - start.tv_nsec);
            if (elapsed > timeout_seconds)
                return NANOEP_ERR_TIMEOUT;
        }
    }
    for (int i = 0; i < NANOEP_HOST_COUNT_WORDS; ++i)
        out[i] = __atomic_load_n(&host_counts[i], __ATOMIC_RELAXED);
    return out[3] != 0 ? NANOEP_ERR_ROUTING : NANOEP_OK;
}

int nanoep_dispatch(const void* x, const float* weights, const int32_t* recv_metadata, const int64_t* dst_slots,
                    const int32_t* token_slots, const int64_t* slot_order, int64_t slot_order_entries,
                    const int64_t* expert_counts, const int64_t* expert_offsets,
                    int64_t recv_count, int64_t expanded_capacity, int64_t num_tokens, int hidden, int num_topk,
                    int64_t num_local_experts, int64_t alignment, int expand, int zero_padding, void* recv_x,
                    int64_t* recv_topk_idx, float* recv_weights, int num_cus, void* stream_handle) {
    if (hidden <= 0 || hidden % 8 != 0 || num_topk <= 0 || num_topk > kMaxTopk || num_local_experts <= 0 || alignment <= 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (recv_count < 0 || num_tokens < 0 || recv_count > num_tokens || num_tokens > INT32_MAX || expanded_capacity < 0 ||
        expanded_capacity > INT32_MAX)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (expand && recv_topk_idx != nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (!aligned16(x) || !aligned16(recv_x))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const int budget_status = validate_cu_budget(num_cus);
    if (budget_status != NANOEP_OK)
        return budget_status;
    const int64_t out_rows = expand ? expanded_capacity : recv_count;
    if (recv_count == 0 || out_rows == 0)
        return NANOEP_OK;  // nothing was received: the outputs have no rows to write
    if ((weights == nullptr) != (recv_weights == nullptr))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (x == nullptr || recv_metadata == nullptr || dst_slots == nullptr || recv_x == nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const bool pad = expand && zero_padding && alignment > 1;
    if (pad && (expert_counts == nullptr || expert_offsets == nullptr))
        return NANOEP_ERR_INVALID_ARGUMENT;

    // full list length without its trailing count word
    const int64_t order_bound = nanoep_slot_order_entries(num_tokens, num_topk, num_local_experts) - 1;
    // The walk pays off once every XCD has at least one whole token block of its own; below that
    // the blocks' source rows would be fetched by several XCDs and the token-order walk is faster.
    const int block_tokens = layout_tokens_per_block(num_local_experts);
    const int64_t token_blocks = block_tokens > 0 ? (num_tokens + block_tokens - 1) / block_tokens : 0;
    const int order_switch = env_int("NANOEP_DISPATCH_ORDER", -1);  // 0 / 1 force the walk off / on
    const bool ordered = expand && slot_order != nullptr && order_bound > 0 &&
                         (order_switch < 0 ? token_blocks >= kNumXcds : order_switch != 0);
    if (ordered && (slot_order_entries > order_bound || num_tokens * num_topk >= (int64_t{1} << 31)))
        return NANOEP_ERR_INVALID_ARGUMENT;
    // a negative entry count defers to the count word the layout stored behind the list
    const int64_t* live_count = ordered && slot_order_entries < 0 ? slot_order + order_bound : nullptr;
    if (live_count != nullptr)
        slot_order_entries = order_bound;

    const int vectors = hidden / 8;
    const int chunks = (vectors + kWave - 1) / kWave;
    const RowBlocking blocking = pick_row_blocking(chunks, ordered ? kSlotOrderWalk : expand ? kTokenOrderWalk : kRowCopyWalk);
    const int64_t waves = static_cast<int64_t>(blocking.chunks_per_block) * blocking.rows_per_block;
    const int64_t copy_candidates = ordered ? slot_order_entries : expand ? num_tokens * num_topk : num_tokens;
    const int64_t copy_blocks = (copy_candidates + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
    // No expert's gap exceeds alignment-1 rows, and all gaps together stay below C.
    const int64_t pad_per_expert = !pad ? 0 : (alignment - 1 < expanded_capacity ? alignment - 1 : expanded_capacity);
    const int64_t pad_groups_per_expert = (pad_per_expert + waves - 1) / waves;
    const int64_t pad_blocks = num_local_experts * pad_groups_per_expert;
    if (copy_candidates >= (int64_t{1} << 31) || copy_blocks + pad_blocks >= (int64_t{1} << 31) - 2 * kNumXcds)
        return NANOEP_ERR_INVALID_ARGUMENT;
    const uint32_t copy_per_xcd = static_cast<uint32_t>((copy_blocks + kNumXcds - 1) / kNumXcds);
    const uint32_t pad_per_xcd = static_cast<uint32_t>((pad_blocks + kNumXcds - 1) / kNumXcds);
    int topk_shift = -1;
    if ((num_topk & (num_topk - 1)) == 0)
        for (topk_shift = 0; (1 << topk_shift) < num_topk; ++topk_shift) {
        }

    const dim3 grid((copy_per_xcd + pad_per_xcd) * kNumXcds);
    const dim3 block(kWave, blocking.chunks_per_block, blocking.rows_per_block);
    const FastDivisor parts_divisor = make_fast_divisor(blocking.parts);
    auto stream = static_cast<hipStream_t>(stream_handle);
    if (ordered) {
        const FastDivisor topk_divisor = make_fast_divisor(static_cast<uint32_t>(num_topk));
#define NANOEP_LAUNCH_ORDERED(DEVICE_COUNT, ZERO_FILL)                                                                \
    dispatch_ordered_kernel<DEVICE_COUNT, ZERO_FILL><<<grid, block, 0, stream>>>(                                    \
        static_cast<const u32x4*>(x), weights, slot_order, live_count, expert_counts, expert_offsets,                \
        static_cast<u32x4*>(recv_x), recv_weights, static_cast<uint32_t>(copy_candidates),                           \
        static_cast<uint32_t>(num_tokens * num_topk), static_cast<uint32_t>(out_rows),                               \
        static_cast<uint32_t>(copy_blocks), copy_per_xcd, static_cast<uint32_t>(pad_blocks), pad_per_xcd,            \
        static_cast<uint32_t>(pad_per_expert),                                                                       \
        static_cast<uint32_t>(pad_groups_per_expert > 0 ? pad_groups_per_expert : 1), blocking.parts,                \
        parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block,                \
        static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), topk_divisor.magic, topk_divisor.shift)
        if (live_count != nullptr && pad_blocks > 0)
            NANOEP_LAUNCH_ORDERED(true, true);
        else if (live_count != nullptr)
            NANOEP_LAUNCH_ORDERED(true, false);
        else if (pad_blocks > 0)
            NANOEP_LAUNCH_ORDERED(false, true);
        else
            NANOEP_LAUNCH_ORDERED(false, false);
#undef NANOEP_LAUNCH_ORDERED
    } else if (!expand) {
        const int64_t blocks = (num_tokens + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
        dispatch_compact_kernel<<<dim3(static_cast<unsigned>(blocks)), block, 0, stream>>>(
            static_cast<const u32x4*>(x), weights, recv_metadata, dst_slots, static_cast<u32x4*>(recv_x), recv_topk_idx,
            recv_weights, static_cast<uint32_t>(num_tokens), static_cast<uint32_t>(recv_count), blocking.parts,
            parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block,
            static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), static_cast<uint32_t>(num_topk));
    } else {
#define NANOEP_LAUNCH_ROWS(LOOKUP, ZERO_FILL)                                                                         \
    dispatch_rows_kernel<LOOKUP, ZERO_FILL><<<grid, block, 0, stream>>>(                                             \
        static_cast<const u32x4*>(x), weights, recv_metadata, dst_slots, token_slots, expert_counts, expert_offsets, \
        static_cast<u32x4*>(recv_x), recv_topk_idx, recv_weights, recv_count, out_rows,                              \
        static_cast<uint32_t>(copy_candidates), static_cast<uint32_t>(copy_blocks), copy_per_xcd,                    \
        static_cast<uint32_t>(pad_blocks), pad_per_xcd, blocking.parts, parts_divisor.magic, parts_divisor.shift,    \
        blocking.chunks_per_block, blocking.rows_per_block, static_cast<uint32_t>(pad_per_expert),                   \
        static_cast<uint32_t>(pad_groups_per_expert > 0 ? pad_groups_per_expert : 1), vectors, chunks, num_topk,     \
        topk_shift, expand ? 1 : 0)
        const bool table = token_slots != nullptr && expand;
        if (table && pad_blocks > 0)
            NANOEP_LAUNCH_ROWS(kLookupTable, true);
        else if (table)
            NANOEP_LAUNCH_ROWS(kLookupTable, false);
        else if (pad_blocks > 0)
            NANOEP_LAUNCH_ROWS(kLookupMetadata, true);
        else
            NANOEP_LAUNCH_ROWS(kLookupMetadata, false);
#undef NANOEP_LAUNCH_ROWS
    }
    NANOEP_HIP_TRY(hipGetLastError());
    return NANOEP_OK;
}

int nanoep_combine(const void* y, const float* weights, const void* bias, const int32_t* recv_metadata,
                   const int64_t* dst_slots, const int32_t* token_slots, int64_t recv_count, int64_t y_rows,
                   int64_t num_tokens, int hidden, int num_topk, int expand, int multiple_reduction, void* out_x,
                   float* out_weights, int num_cus, void* stream_handle) {
    if (hidden <= 0 || hidden % 8 != 0 || num_topk <= 0 || num_topk > kMaxTopk)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (recv_count < 0 || num_tokens < 0 || recv_count > num_tokens || num_tokens > INT32_MAX || y_rows < 0 ||
        y_rows > INT32_MAX)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (!expand && y_rows != recv_count)
        return NANOEP_ERR_INVALID_ARGUMENT;
    // weights may be a null pointer only when it has no rows (nothing was received)
    if ((weights != nullptr && out_weights == nullptr) || (weights == nullptr && out_weights != nullptr && y_rows > 0))
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (!aligned16(y) || !aligned16(out_x) || !aligned16(bias))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const int budget_status = validate_cu_budget(num_cus);
    if (budget_status != NANOEP_OK)
        return budget_status;
    if (num_tokens == 0)
        return NANOEP_OK;
    if (out_x == nullptr || dst_slots == nullptr || (recv_count > 0 && (recv_metadata == nullptr || y == nullptr)))
        return NANOEP_ERR_INVALID_ARGUMENT;

    const int vectors = hidden / 8;
    const int chunks = (vectors + kWave - 1) / kWave;
    const RowBlocking blocking = pick_row_blocking(chunks, expand ? kTokenOrderWalk : kRowCopyWalk);
    const int64_t blocks = (num_tokens + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
    if (blocks >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const dim3 grid(static_cast<unsigned>(blocks));
    const dim3 block(kWave, blocking.chunks_per_block, blocking.rows_per_block);
    auto stream = static_cast<hipStream_t>(stream_handle);
    const int gathered = expand ? num_topk : 1;
    // the slot table only helps the expanded layout, and only when something was received
    const bool direct = token_slots != nullptr && expand && recv_count > 0;
    const FastDivisor parts_divisor = make_fast_divisor(blocking.parts);
    if (!expand) {
        // y may be a null pointer when nothing was received: every token then takes the hole path
        combine_compact_kernel<<<grid, block, 0, stream>>>(
            static_cast<const u32x4*>(recv_count > 0 ? y : out_x), weights, static_cast<const u32x4*>(bias), recv_metadata,
            dst_slots, static_cast<u32x4*>(out_x), out_weights, static_cast<uint32_t>(num_tokens),
            static_cast<uint32_t>(recv_count), blocking.parts, parts_divisor.magic, parts_divisor.shift,
            blocking.chunks_per_block, blocking.rows_per_block, static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks),
            static_cast<uint32_t>(num_topk));
        NANOEP_HIP_TRY(hipGetLastError());
        return NANOEP_OK;
    }
    if (direct && num_topk >= 2 && num_topk <= 4) {
#define NANOEP_LAUNCH_FEW(TOPK)                                                                                       \
    combine_few_rows_kernel<TOPK><<<grid, block, 0, stream>>>(                                                       \
        static_cast<const u32x4*>(y), weights, static_cast<const u32x4*>(bias), token_slots,                         \
        static_cast<u32x4*>(out_x), out_weights, static_cast<uint32_t>(num_tokens), static_cast<uint32_t>(y_rows),   \
        blocking.parts, parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block, \
        static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), static_cast<uint32_t>(num_topk),              \
        multiple_reduction ? 1 : 0)
        if (num_topk == 2)
            NANOEP_LAUNCH_FEW(2);
        else
            NANOEP_LAUNCH_FEW(4);
#undef NANOEP_LAUNCH_FEW
        NANOEP_HIP_TRY(hipGetLastError());
        return NANOEP_OK;
    }
#define NANOEP_LAUNCH_COMBINE(GROUP, DIRECT)                                                                       \
    combine_rows_kernel<GROUP, DIRECT><<<grid, block, 0, stream>>>(                                                \
        static_cast<const u32x4*>(y), weights, static_cast<const u32x4*>(bias), recv_metadata, dst_slots,          \
        token_slots, static_cast<u32x4*>(out_x), out_weights, recv_count, y_rows, static_cast<uint32_t>(num_tokens), \
        blocking.parts, parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block,  \
        vectors, chunks, num_topk, expand ? 1 : 0,                                                                   \
        multiple_reduction ? 1 : 0)
#define NANOEP_LAUNCH_COMBINE_GROUP(GROUP)    \
    do {                                     \
        if (direct)                          \
            NANOEP_LAUNCH_COMBINE(GROUP, true);  \
        else                                 \
            NANOEP_LAUNCH_COMBINE(GROUP, false); \
    } while (0)
    // the group size is the number of rows fetched per pass: the smallest of 1, 2, 4, 8, 16 covering K
    if (gathered <= 1)
        NANOEP_LAUNCH_COMBINE_GROUP(1);
    else if (gathered <= 2)
        NANOEP_LAUNCH_COMBINE_GROUP(2);
    else if (gathered <= 4)
        NANOEP_LAUNCH_COMBINE_GROUP(4);
    else if (gathered <= 8)
        NANOEP_LAUNCH_COMBINE_GROUP(8);
    else
        NANOEP_LAUNCH_COMBINE_GROUP(16);
#undef NANOEP_LAUNCH_COMBINE_GROUP
#undef NANOEP_LAUNCH_COMBINE
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
