// Dispatch permute / expand: slot-order walk, token-order walks, compact row copy, zero fill.

#include "nanoep_device.h"

namespace nanoep {
namespace {

// One wavefront moves one 1 KiB chunk (64 lanes x 16 bytes) of one destination row with exactly
// one 128-bit load and one nontemporal 128-bit store per lane: on this part a wavefront that issues
// a single store and retires sustains more HBM write bandwidth than one that issues several.
//
// A workgroup is (64, chunks_per_block, rows_per_block): threadIdx.y is the chunk, threadIdx.z the
// destination candidate, so no per-wave division by the chunk count is needed.  In the token-order
// walk of the expanded layout (dispatch_rows_kernel) candidates are ordered (source token, k): the K destinations of a token are handled by consecutive workgroups
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
    if (out_row < 0 || out_row >= uniform_load(expert_offsets + expert + 1) || out_row >= out_rows)
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
                                                             u32x4* __restrict__ recv_x,                // [C][vectors]
                                                             float* __restrict__ recv_weights,          // [C] or null
                                                             int64_t recv_count,
                                                             int64_t out_rows,
                                                             uint32_t copy_candidates,  // T*K
                                                             uint32_t copy_blocks,
                                                             uint32_t copy_per_xcd,  // ceil(copy_blocks / XCDs)
                                                             uint32_t pad_blocks,
                                                             uint32_t pad_per_xcd,   // ceil(pad_blocks / XCDs)
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
                                                             XcdMap xcds) {
    NANOEP_FETCH_ARGS_4(x, weights, recv_x, recv_weights);
    NANOEP_FETCH_ARGS_4(token_slots, copy_blocks, dst_slots, recv_metadata);
    NANOEP_FETCH_ARGS_4(out_rows, recv_count, copy_candidates, copy_per_xcd);
    NANOEP_FETCH_ARGS_4(parts_magic, parts_shift, vectors, chunks);
    NANOEP_FETCH_ARGS_4(num_topk, topk_shift, rows_per_block, chunks_per_block);
    NANOEP_FETCH_ARGS_4(xcds.count, xcds.magic, xcds.shift, copy_per_xcd);
    // Workgroups are handed to the XCDs round-robin.  Each XCD takes one contiguous range of the
    // copy work followed by one contiguous range of the zero-fill work, so neighbouring work items
    // (which share their source rows) stay behind one L2 and every XCD gets its share of both.
    // (kZeroFill is false when the launch has no zero-fill work: the copy path then carries none of
    // its bookkeeping, which shows in a wavefront that lives about a microsecond)
    const uint32_t index_in_xcd = fast_divide(blockIdx.x, xcds.magic, xcds.shift);
    const uint32_t xcd = blockIdx.x - index_in_xcd * xcds.count;
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
        // candidates are (source token, k) pairs in token order
        uint32_t token = topk_shift >= 0 ? candidate >> topk_shift : candidate / static_cast<uint32_t>(num_topk);
        int k = static_cast<int>(candidate - token * num_topk);
        token = __builtin_amdgcn_readfirstlane(token);
        k = __builtin_amdgcn_readfirstlane(k);
        // lanes past the end of a short row re-read vector 0 instead of branching around the load
        const u32x4 data = x[static_cast<int64_t>(token) * vectors + (in_row ? vector : 0)];
        int64_t out_row;
        if (kLookup == kLookupTable) {
            out_row = uniform_load(token_slots + static_cast<int64_t>(token) * num_topk + k);
        } else {
            const int64_t row = uniform_load(dst_slots + token);
            if (row < 0 || row >= recv_count)
                return;
            out_row = static_cast<int64_t>(uniform_load(recv_metadata + row * (num_topk + 2) + 2 + k));
        }
        if (out_row < 0 || out_row >= out_rows)
            return;
        if (in_row)
            store_vec<true>(recv_x + out_row * vectors + vector, data);
        if (chunk == 0 && lane == 0 && recv_weights != nullptr)
            recv_weights[out_row] = weights[static_cast<int64_t>(token) * num_topk + k];
    } else {
        zero_fill_gap_rows(block, pad_per_expert, pad_groups_per_expert, chunks_per_block, rows_per_block, expert_counts,
                           expert_offsets, recv_x, recv_weights, out_rows, vectors);
    }
}

// The slot-order walk, stripped to what its wavefronts need: a wavefront lives about a microsecond,
// most of it waiting in a chain of scalar work -> list entry -> source load -> store, so every
// scalar instruction and branch ahead of the source load is throughput (ten more scalar
// instructions and three taken branches there measured +6 % on the whole kernel).  kZeroFill is
// false when the launch has no gap rows to clear: the copy path then carries none of that
// bookkeeping.  kWholeRows is the launch with one workgroup a list entry and one wavefront a piece
// of the row (rows of 5 to 16 pieces, no side workgroups): block index and wavefront index are
// the entry and the piece, with no division and no taken branch on the way to the load.
// kSpan is the number of consecutive 1 KiB chunks a wavefront moves (loads issued back to back,
// then the stores).  One is best while the source fits the last-level cache; beyond that size the
// single-chunk walk loses a quarter of its rate and two chunks a wavefront win it back.
// kPrefetch: the list is cut into segments of about one window's entries, and the copy workgroups of
// every segment are preceded by a few workgroups that read the window's source rows front to back
// (kPrefetchLoads KiB a wavefront, the data dropped).  The window's first touches then reach HBM as
// one sequential burst ahead of the segment's stores instead of one row at a time among them, and
// the copy wavefronts find their rows in the XCD's L2.  No bytes are read twice from HBM; what it
// costs is one more L2 read per source row.
constexpr int kPrefetchLoads = 4;

template <bool kDeviceCount, bool kZeroFill, int kSpan, bool kWholeRows, bool kPrefetch>
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
                                                                uint32_t chunks,      // pieces of kSpan chunks in a row
                                                                uint32_t topk_magic,  // fast divisor by K
                                                                uint32_t topk_shift,
                                                                uint32_t rows_magic,  // fast divisor by rows_per_block
                                                                uint32_t rows_shift,
                                                                uint32_t payload_blocks,  // blocks behind them, if any, move the weights
                                                                uint32_t segment_blocks,     // kPrefetch: prefetch + copy workgroups of a segment
                                                                uint32_t segment_magic,      // fast divisor by segment_blocks
                                                                uint32_t segment_shift,
                                                                uint32_t prefetch_blocks,    // prefetch workgroups at the head of a segment
                                                                uint32_t share_magic,        // fast divisor by the copy workgroups of a segment
                                                                uint32_t share_shift,
                                                                uint32_t window_vectors,     // 16-byte vectors of one window's source rows
                                                                uint32_t source_vectors,     // ... of all source rows
                                                                XcdMap xcds) {
    NANOEP_FETCH_ARGS_4(x, weights, recv_x, recv_weights);
    NANOEP_FETCH_ARGS_4(slot_order, entries, source_limit, out_rows);
    NANOEP_FETCH_ARGS_4(copy_blocks, copy_per_xcd, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    NANOEP_FETCH_ARGS_4(chunks, topk_magic, topk_shift, live_count);
    NANOEP_FETCH_ARGS_4(xcds.count, xcds.magic, xcds.shift, payload_blocks);
    // workgroups per XCD the grid holds for the copy work: with the entry count on the device the live
    // list may be shorter (the rest of the grid leaves at once) or longer (workgroups then take more
    // than one turn, `grid_copy_per_xcd` list positions apart) than what the grid was sized for
    const uint32_t grid_copy_per_xcd = copy_per_xcd;
    if (kDeviceCount) {
        // The list length was not known when the grid was sized: the walk covers the entries in use,
        // so that the per-XCD ranges split the real work and not an unused tail.
        // A word that cannot be a count (the layout did not run) walks nothing.
        const int64_t live = uniform_load(live_count);
        entries = live >= 0 && live <= static_cast<int64_t>(source_limit) ? static_cast<uint32_t>(live) : 0u;
        // (one workgroup a list entry: no division by a runtime number on every wavefront's way to its load)
        if (kWholeRows)
            copy_blocks = entries;
        else
            copy_blocks = fast_divide(entries + rows_per_block - 1, rows_magic, rows_shift) * parts;
        // with prefetch: whole segments of the size the host chose (from the count it expected), each
        // with its prefetch workgroups in front
        const uint32_t walk_blocks =
            kPrefetch ? fast_divide(copy_blocks + (segment_blocks - prefetch_blocks) - 1, share_magic, share_shift) * segment_blocks
                      : copy_blocks;
        copy_per_xcd = fast_divide(walk_blocks + xcds.count - 1, xcds.magic, xcds.shift);
    }
    if (!kWholeRows && blockIdx.x >= payload_blocks) {
        // The weights of the assignments, one lane per list entry, in workgroups of their own at the
        // end of the grid.  The host asks for them when a row is one or two chunks: hung onto the
        // row's first payload wavefront the weight is a second round trip in every (second) wavefront
        // (131072 x 512 top-8: 77.5 -> 74.5 us).  With longer rows the first wavefronts are few and
        // carry it at no measurable cost, while these extra workgroups cost 0.1 ns per assignment
        // (4096 x 7168: +1 us, 32768 x 7168: +25 us of 700).
        const uint32_t wave = threadIdx.z * chunks_per_block + threadIdx.y;
        const uint32_t lanes = (gridDim.x - payload_blocks) * (chunks_per_block * rows_per_block) * kWave;
        for (uint32_t flat = ((blockIdx.x - payload_blocks) * (chunks_per_block * rows_per_block) + wave) * kWave + threadIdx.x;
             flat < entries; flat += lanes) {
            const int64_t entry = slot_order[flat];
            const uint32_t source = static_cast<uint32_t>(entry);
            const uint32_t out_row = static_cast<uint32_t>(static_cast<uint64_t>(entry) >> 32);
            if (entry >= 0 && source < source_limit && out_row < out_rows)
                recv_weights[out_row] = weights[source];
        }
        return;
    }
    const uint32_t index_in_xcd = fast_divide(blockIdx.x, xcds.magic, xcds.shift);
    const uint32_t xcd = blockIdx.x - index_in_xcd * xcds.count;
    // the XCD's workgroups up to `copy_turns` copy, the ones behind them clear gap rows
    const uint32_t copy_turns = kDeviceCount && copy_per_xcd > grid_copy_per_xcd ? grid_copy_per_xcd : copy_per_xcd;
    if (kZeroFill && index_in_xcd >= copy_turns) {
        const uint32_t pad_index = index_in_xcd - copy_turns;
        const uint32_t pad_block = xcd * pad_per_xcd + pad_index;
        if (pad_index < pad_per_xcd && pad_block < pad_blocks)
            zero_fill_gap_rows(pad_block, pad_per_expert, pad_groups_per_expert, chunks_per_block, rows_per_block,
                               expert_counts, expert_offsets, recv_x, recv_weights, out_rows, static_cast<int>(vectors));
        return;
    }
    if (index_in_xcd >= copy_turns)
        return;
    // one turn, except where a device-side count found more entries than the grid was sized for
    for (uint32_t at = index_in_xcd; at < copy_per_xcd; at += grid_copy_per_xcd) {
        uint32_t block = xcd * copy_per_xcd + at;
        if (kPrefetch) {
            const uint32_t segment = fast_divide(block, segment_magic, segment_shift);
            const uint32_t within = block - segment * segment_blocks;
            if (within < prefetch_blocks) {
                const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.z * chunks_per_block + threadIdx.y);
                const uint32_t waves = chunks_per_block * rows_per_block;
                const uint64_t window_first = static_cast<uint64_t>(segment) * window_vectors;
                uint64_t window_end = window_first + window_vectors;
                if (window_end > source_vectors)
                    window_end = source_vectors;
                const uint64_t first = window_first + static_cast<uint64_t>(within * waves + wave) * (kPrefetchLoads * kWave);
                if (first < window_end) {
                    u32x4 fetched[kPrefetchLoads];
#pragma unroll
                    for (int u = 0; u < kPrefetchLoads; ++u) {
                        const uint64_t from = first + u * kWave + threadIdx.x;
                        fetched[u] = x[from < window_end ? from : window_first];
                    }
#pragma unroll
                    for (int u = 0; u < kPrefetchLoads; ++u)
                        asm volatile("" ::"v"(fetched[u].x), "v"(fetched[u].y), "v"(fetched[u].z), "v"(fetched[u].w));
                }
                if (!kDeviceCount)
                    break;
                continue;
            }
            block = segment * (segment_blocks - prefetch_blocks) + (within - prefetch_blocks);
        }
        uint32_t candidate, chunk;
        if (kWholeRows) {
            // one workgroup a row, as many wavefronts as the row has pieces: the block is the list entry
            if (block >= entries)
                break;
            candidate = block;
            chunk = __builtin_amdgcn_readfirstlane(threadIdx.y);
        } else {
            if (block >= copy_blocks)
                break;
            const uint32_t group = fast_divide(block, parts_magic, parts_shift);
            const uint32_t part = block - group * parts;
            candidate = group * rows_per_block + __builtin_amdgcn_readfirstlane(threadIdx.z);
            chunk = part * chunks_per_block + __builtin_amdgcn_readfirstlane(threadIdx.y);
        }
        if (kWholeRows || (candidate < entries && chunk < chunks)) {
            const int64_t entry = uniform_load(slot_order + candidate);
            const uint32_t source = static_cast<uint32_t>(entry);
            const uint32_t out_row = static_cast<uint32_t>(static_cast<uint64_t>(entry) >> 32);
            if (entry >= 0 && source < source_limit && out_row < out_rows) {
                const uint32_t token = fast_divide(source, topk_magic, topk_shift);
                const uint32_t vector = chunk * (kSpan * kWave) + threadIdx.x;
                // no workgroups behind the payload: the row's first wavefront moves its weight, fetched through
                // the scalar path while the payload load is in flight
                const bool carries_weight = chunk == 0 && recv_weights != nullptr && (kWholeRows || payload_blocks == gridDim.x);
                float weight = 0.0f;
                if (carries_weight)
                    weight = uniform_load(weights + source);
                u32x4 data[kSpan];
#pragma unroll
                for (int s = 0; s < kSpan; ++s) {
                    const uint32_t from = vector + s * kWave;
                    data[s] = x[static_cast<uint64_t>(token) * vectors + (from < vectors ? from : 0u)];
                }
#pragma unroll
                for (int s = 0; s < kSpan; ++s) {
                    const uint32_t to = vector + s * kWave;
                    if (to < vectors)
                        store_vec<true>(recv_x + static_cast<uint64_t>(out_row) * vectors + to, data[s]);
                }
                if (carries_weight && threadIdx.x == 0)
                    recv_weights[out_row] = weight;
            }
        }
        if (!kDeviceCount)
            break;
    }
}

// Compact layout: receive row r holds source token src_token(r), in token order, so the dispatch is
// a row copy with holes.  Nothing is re-used, so workgroups walk the rows in plain launch order
// (one linear stream over the whole device) and the payload wavefronts carry nothing but the copy.
// The rows' ids and weights are moved by `side_blocks` workgroups of their own at the front of the
// grid, one lane per (token, k): hung onto the first payload wavefront of every row they cost 11 us
// of a 95 us kernel at 32768 x 4096, top-8 (two more dependent round trips in one wavefront in
// eight); on their own, with full wavefronts and coalesced rows, next to nothing.
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
                                                                uint32_t topk,
                                                                uint32_t topk_magic,  // fast divisor by K
                                                                uint32_t topk_shift,
                                                                uint32_t side_blocks) {
    NANOEP_FETCH_ARGS_4(x, dst_slots, recv_x, tokens);
    NANOEP_FETCH_ARGS_4(recv_count, parts, parts_magic, parts_shift);
    NANOEP_FETCH_ARGS_4(chunks_per_block, rows_per_block, vectors, chunks);
    if (blockIdx.x < side_blocks) {
        const uint32_t wave = threadIdx.z * chunks_per_block + threadIdx.y;
        const uint32_t flat = (blockIdx.x * (chunks_per_block * rows_per_block) + wave) * kWave + threadIdx.x;
        const uint32_t token = fast_divide(flat, topk_magic, topk_shift);
        if (token >= tokens)
            return;
        const uint32_t k = flat - token * topk;
        const int64_t row = dst_slots[token];
        if (row < 0 || row >= static_cast<int64_t>(recv_count))
            return;
        if (recv_topk_idx != nullptr)
            recv_topk_idx[row * topk + k] = recv_metadata[row * (topk + 2) + 2 + k];
        if (recv_weights != nullptr)
            recv_weights[row * topk + k] = weights[flat];
        return;
    }
    const uint32_t payload_block = blockIdx.x - side_blocks;
    const uint32_t group = fast_divide(payload_block, parts_magic, parts_shift);
    const uint32_t part = payload_block - group * parts;
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
}


}  // namespace
}  // namespace nanoep

using namespace nanoep;

extern "C" {

int nanoep_dispatch(const void* x, const float* weights, const int32_t* recv_metadata, const int64_t* dst_slots,
                    const int32_t* token_slots, const int64_t* slot_order, int64_t slot_order_entries,
                    const int64_t* expert_counts, const int64_t* expert_offsets,
                    int64_t recv_count, int64_t expanded_capacity, int64_t num_tokens, int hidden, int num_topk,
                    int64_t num_local_experts, int64_t alignment, int expand, int zero_padding, void* recv_x,
                    int64_t* recv_topk_idx, float* recv_weights, int num_cus, void* stream_handle) {
    const Tuning tuning = current_tuning();
    if (hidden <= 0 || hidden % 8 != 0 || num_topk <= 0 || num_topk > kMaxTopk || num_local_experts <= 0 || alignment <= 0)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (recv_count < 0 || num_tokens < 0 || recv_count > num_tokens || num_tokens > INT32_MAX || expanded_capacity < 0 ||
        expanded_capacity > INT32_MAX)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (expand && recv_topk_idx != nullptr)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (!aligned16(x) || !aligned16(recv_x))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const Topology topology = current_topology(tuning);
    const int budget_status = validate_cu_budget(num_cus, topology);
    if (budget_status != NANOEP_OK)
        return budget_status;
    const XcdMap xcds = make_xcd_map(topology.xcds);
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
    // The walk is used whenever the handle carries the list.  With cache-resident sources and fewer
    // than eight token blocks the token-order walk is up to 15 % faster, but with cold sources it is
    // 25-60 % slower at every size, so the list decides.
    const int order_switch = tuning.dispatch_order;  // 0 forces the token-order walk
    const bool ordered = expand && slot_order != nullptr && order_bound > 0 && order_switch != 0;
    if (ordered && (slot_order_entries > order_bound || num_tokens * num_topk >= (int64_t{1} << 31)))
        return NANOEP_ERR_INVALID_ARGUMENT;
    // A negative entry count defers to the count word the layout stored behind the list.  -1 sizes the
    // grid for the most entries the list can hold (T * K), -g for about g of them: workgroups beyond
    // the live count leave at once, and where the live count is above g workgroups take several turns.
    const int64_t* live_count = ordered && slot_order_entries < 0 ? slot_order + order_bound : nullptr;
    if (live_count != nullptr) {
        const int64_t most = num_tokens * num_topk;
        const int64_t expected = slot_order_entries == -1 ? most : -slot_order_entries;
        slot_order_entries = expected < most ? expected : most;
    }

    const int vectors = hidden / 8;
    int chunks = (vectors + kWave - 1) / kWave;
    // Chunks per wavefront of the slot-order walk: two once the source outgrows the last-level cache,
    // and for rows of two chunks, which then take one wavefront (16384 x 1024 top-4: 39.8 -> 35.6 us;
    // at four chunks the gain is within +3 / -1 %).  NANOEP_DISPATCH_SPAN=1|2 overrides.  `chunks`
    // then counts pieces of that many chunks.
    const int row_chunks = chunks;
    int span = 1;
    if (ordered) {
        const bool short_rows = chunks == 2;
        span = short_rows || static_cast<int64_t>(num_tokens) * hidden * 2 > kLastLevelCacheBytes ? 2 : 1;
        const int forced_span = tuning.dispatch_span;
        if (forced_span == 1 || forced_span == 2)
            span = forced_span;
        chunks = (chunks + span - 1) / span;
    }
    const WalkShape walk = ordered ? kSlotOrderWalk : expand ? kTokenOrderWalk : kRowCopyWalk;
    const RowBlocking blocking = pick_row_blocking(chunks, walk, tuning);
    const int64_t waves = static_cast<int64_t>(blocking.chunks_per_block) * blocking.rows_per_block;
    const int64_t copy_candidates = ordered ? slot_order_entries : expand ? num_tokens * num_topk : num_tokens;
    const int64_t copy_blocks = (copy_candidates + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
    // No expert's gap exceeds alignment-1 rows, and all gaps together stay below C.
    const int64_t pad_per_expert = !pad ? 0 : (alignment - 1 < expanded_capacity ? alignment - 1 : expanded_capacity);
    const int64_t pad_groups_per_expert = (pad_per_expert + waves - 1) / waves;
    const int64_t pad_blocks = num_local_experts * pad_groups_per_expert;
    if (copy_candidates >= (int64_t{1} << 31) || copy_blocks + pad_blocks >= (int64_t{1} << 31) - 2 * int64_t{xcds.count})
        return NANOEP_ERR_INVALID_ARGUMENT;
    // Prefetch workgroups ahead of every window's share of the list.  The list's windows hold nearly the same number of entries each, so equal shares
    // of the list follow them closely.
    const int window_tokens = ordered ? nanoep_layout_block_tokens(num_tokens, num_local_experts, hidden) : 0;
    // On by default for rows of two chunks (513 to 1024 elements), where it gains 7 to 19 % with sources
    // that come from HBM and costs nothing with cache-resident ones.  For other row lengths it trades:
    // rows of one chunk +21 % against -14 %, the 4096 x 4096 top-2 batch +7 % against -9 %, rows of 7168
    // elements +0 to 2 % against -10 %; there it is the caller's choice (the DISPATCH_PREFETCH switch).
    const bool prefetch = ordered && window_tokens > 0 && copy_blocks > 0 &&
                          (tuning.dispatch_prefetch < 0 ? row_chunks == 2 : tuning.dispatch_prefetch > 0);
    int64_t segment_copy_blocks = 0, segment_prefetch_blocks = 0, segments = 0;
    if (prefetch) {
        const int64_t windows = (num_tokens + window_tokens - 1) / window_tokens;
        const int64_t segment_entries = (copy_candidates + windows - 1) / windows;
        segment_copy_blocks = (segment_entries + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
        segments = (copy_blocks + segment_copy_blocks - 1) / segment_copy_blocks;
        const int64_t window_kib = (static_cast<int64_t>(window_tokens) * vectors + kWave - 1) / kWave;
        segment_prefetch_blocks = (window_kib + waves * kPrefetchLoads - 1) / (waves * kPrefetchLoads);
    }
    const int64_t walk_blocks = prefetch ? segments * (segment_copy_blocks + segment_prefetch_blocks) : copy_blocks;
    if (walk_blocks >= (int64_t{1} << 31) - 2 * int64_t{xcds.count} - pad_blocks ||
        static_cast<int64_t>(num_tokens) * vectors >= (int64_t{1} << 32))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const uint32_t copy_per_xcd = static_cast<uint32_t>((walk_blocks + xcds.count - 1) / xcds.count);
    const uint32_t pad_per_xcd = static_cast<uint32_t>((pad_blocks + xcds.count - 1) / xcds.count);
    int topk_shift = -1;
    if ((num_topk & (num_topk - 1)) == 0)
        for (topk_shift = 0; (1 << topk_shift) < num_topk; ++topk_shift) {
        }

    // slot-order walk over rows of one or two chunks: one lane per list entry moves the weights, in
    // workgroups at the end of the grid (+3-4 %); longer rows carry the weight on their first wavefront
    // (8192 x 2048 top-8 with alignment 128: 56.0 against 57.0 us).  NANOEP_DISPATCH_SIDE=0|1 overrides.
    const int side_switch = tuning.dispatch_side;
    const bool side_weights = ordered && recv_weights != nullptr && (side_switch < 0 ? row_chunks <= 2 : side_switch != 0);
    const int64_t side_lanes = side_weights ? copy_candidates : 0;
    const int64_t side_blocks = (side_lanes + kWave * waves - 1) / (kWave * waves);
    const int64_t payload_blocks = (int64_t{copy_per_xcd} + pad_per_xcd) * xcds.count;
    if (payload_blocks + side_blocks >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const dim3 grid(static_cast<unsigned>(payload_blocks + side_blocks));
    const dim3 block(kWave, blocking.chunks_per_block, blocking.rows_per_block);
    const FastDivisor parts_divisor = make_fast_divisor(blocking.parts);
    auto stream = static_cast<hipStream_t>(stream_handle);
    if (ordered) {
        const FastDivisor topk_divisor = make_fast_divisor(static_cast<uint32_t>(num_topk));
        const FastDivisor rows_divisor = make_fast_divisor(blocking.rows_per_block);
        const FastDivisor share_divisor = make_fast_divisor(static_cast<uint32_t>(prefetch ? segment_copy_blocks : 1));
        const FastDivisor segment_divisor = make_fast_divisor(static_cast<uint32_t>(prefetch ? segment_copy_blocks + segment_prefetch_blocks : 1));
#define NANOEP_LAUNCH_ORDERED_ROWS(DEVICE_COUNT, ZERO_FILL, SPAN, WHOLE_ROWS, PREFETCH)                               \
    dispatch_ordered_kernel<DEVICE_COUNT, ZERO_FILL, SPAN, WHOLE_ROWS, PREFETCH><<<grid, block, 0, stream>>>(        \
        static_cast<const u32x4*>(x), weights, slot_order, live_count, expert_counts, expert_offsets,                \
        static_cast<u32x4*>(recv_x), recv_weights, static_cast<uint32_t>(copy_candidates),                           \
        static_cast<uint32_t>(num_tokens * num_topk), static_cast<uint32_t>(out_rows),                               \
        static_cast<uint32_t>(copy_blocks), copy_per_xcd, static_cast<uint32_t>(pad_blocks), pad_per_xcd,            \
        static_cast<uint32_t>(pad_per_expert),                                                                       \
        static_cast<uint32_t>(pad_groups_per_expert > 0 ? pad_groups_per_expert : 1), blocking.parts,                \
        parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block,                \
        static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), topk_divisor.magic, topk_divisor.shift,       \
        rows_divisor.magic, rows_divisor.shift, static_cast<uint32_t>(payload_blocks),                               \
        static_cast<uint32_t>(segment_copy_blocks + segment_prefetch_blocks), segment_divisor.magic,                 \
        segment_divisor.shift, static_cast<uint32_t>(segment_prefetch_blocks),                                       \
        share_divisor.magic, share_divisor.shift,                                                                    \
        static_cast<uint32_t>(static_cast<int64_t>(window_tokens) * vectors),                                        \
        static_cast<uint32_t>(num_tokens * vectors), xcds)
#define NANOEP_LAUNCH_ORDERED_SPAN(DEVICE_COUNT, ZERO_FILL, SPAN)                                 \
    do {                                                                                          \
        if (whole_rows && prefetch)                                                               \
            NANOEP_LAUNCH_ORDERED_ROWS(DEVICE_COUNT, ZERO_FILL, SPAN, true, true);                \
        else if (whole_rows)                                                                      \
            NANOEP_LAUNCH_ORDERED_ROWS(DEVICE_COUNT, ZERO_FILL, SPAN, true, false);               \
        else if (prefetch)                                                                        \
            NANOEP_LAUNCH_ORDERED_ROWS(DEVICE_COUNT, ZERO_FILL, SPAN, false, true);               \
        else                                                                                      \
            NANOEP_LAUNCH_ORDERED_ROWS(DEVICE_COUNT, ZERO_FILL, SPAN, false, false);              \
    } while (0)
#define NANOEP_LAUNCH_ORDERED(DEVICE_COUNT, ZERO_FILL)             \
    do {                                                           \
        if (span == 2)                                             \
            NANOEP_LAUNCH_ORDERED_SPAN(DEVICE_COUNT, ZERO_FILL, 2); \
        else                                                       \
            NANOEP_LAUNCH_ORDERED_SPAN(DEVICE_COUNT, ZERO_FILL, 1); \
    } while (0)
        // a workgroup per list entry with a wavefront per piece of the row: the kernel then needs no
        // division to find its entry and piece (4096 x 7168: 81.5 -> 80.4 us, with alignment 128
        // 100.6 -> 96.9 us, 8192 x 5120: 123.1 -> 120.3 us).  Rows of four pieces are better off
        // with the general path (8192 x 2048 with cache-resident sources: 37.6 against 38.3 us).
        const int whole_rows_switch = tuning.dispatch_whole_rows;
        const bool whole_rows = blocking.parts == 1 && blocking.rows_per_block == 1 &&
                                blocking.chunks_per_block == static_cast<unsigned>(chunks) && side_blocks == 0 &&
                                (whole_rows_switch < 0 ? chunks >= 5 : whole_rows_switch != 0);
        if (live_count != nullptr && pad_blocks > 0)
            NANOEP_LAUNCH_ORDERED(true, true);
        else if (live_count != nullptr)
            NANOEP_LAUNCH_ORDERED(true, false);
        else if (pad_blocks > 0)
            NANOEP_LAUNCH_ORDERED(false, true);
        else
            NANOEP_LAUNCH_ORDERED(false, false);
#undef NANOEP_LAUNCH_ORDERED
#undef NANOEP_LAUNCH_ORDERED_SPAN
#undef NANOEP_LAUNCH_ORDERED_ROWS
    } else if (!expand) {
        const int64_t blocks = (num_tokens + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
        // one lane per (token, k) for the ids and weights, when the caller wants either
        const int64_t row_side_lanes = recv_topk_idx != nullptr || recv_weights != nullptr ? num_tokens * num_topk : 0;
        const int64_t row_side_blocks = (row_side_lanes + kWave * waves - 1) / (kWave * waves);
        if (row_side_lanes >= (int64_t{1} << 31) || blocks + row_side_blocks >= (int64_t{1} << 31))
            return NANOEP_ERR_INVALID_ARGUMENT;
        const FastDivisor topk_divisor = make_fast_divisor(static_cast<uint32_t>(num_topk));
        dispatch_compact_kernel<<<dim3(static_cast<unsigned>(blocks + row_side_blocks)), block, 0, stream>>>(
            static_cast<const u32x4*>(x), weights, recv_metadata, dst_slots, static_cast<u32x4*>(recv_x), recv_topk_idx,
            recv_weights, static_cast<uint32_t>(num_tokens), static_cast<uint32_t>(recv_count), blocking.parts,
            parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block,
            static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), static_cast<uint32_t>(num_topk),
            topk_divisor.magic, topk_divisor.shift, static_cast<uint32_t>(row_side_blocks));
    } else {
#define NANOEP_LAUNCH_ROWS(LOOKUP, ZERO_FILL)                                                                         \
    dispatch_rows_kernel<LOOKUP, ZERO_FILL><<<grid, block, 0, stream>>>(                                             \
        static_cast<const u32x4*>(x), weights, recv_metadata, dst_slots, token_slots, expert_counts, expert_offsets, \
        static_cast<u32x4*>(recv_x), recv_weights, recv_count, out_rows,                                             \
        static_cast<uint32_t>(copy_candidates), static_cast<uint32_t>(copy_blocks), copy_per_xcd,                    \
        static_cast<uint32_t>(pad_blocks), pad_per_xcd, blocking.parts, parts_divisor.magic, parts_divisor.shift,    \
        blocking.chunks_per_block, blocking.rows_per_block, static_cast<uint32_t>(pad_per_expert),                   \
        static_cast<uint32_t>(pad_groups_per_expert > 0 ? pad_groups_per_expert : 1), vectors, chunks, num_topk,     \
        topk_shift, xcds)
        const bool table = token_slots != nullptr;
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

}  // extern "C"
