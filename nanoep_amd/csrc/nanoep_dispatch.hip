// Dispatch permute / expand: slot-order walk, token-order walks, compact row copy, zero fill.

#include "nanoep_device.h"

namespace nanoep {
namespace {

// One wavefront moves one 1 KiB chunk (64 lanes x 16 bytes) of one destination row with exactly
// one 128-bit load and one nontemporal 128-bit store per lane: on this part a wavefront that issues
// a single store and retires sustains more HBM write bandwidth than one that issues several.
//
// The token-order walks and the compact row copy use workgroups of (64, chunks_per_block,
// rows_per_block): threadIdx.y is the chunk, threadIdx.z the destination candidate, so no per-wave
// division by the chunk count is needed.  In the token-order walk of the expanded layout
// (dispatch_rows_kernel) candidates are ordered (source token, k): the K destinations of a token are
// handled by consecutive workgroups behind one XCD's L2, so only the first read of a source row goes
// to HBM, and every destination row is written as one contiguous run by the wavefronts of one
// workgroup.  The source address depends only on the block index, so its load is in flight while the
// wave-uniform lookups (token_slots[t][k], or dst_slots[t] -> recv_metadata[row][2+k] for a handle
// without that table) resolve the destination row.  The slot-order walk (dispatch_walk_kernel, further
// down) has one-dimensional workgroups and its own, leaner bookkeeping.
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

// Arguments of dispatch_walk_kernel.  The first words are what every copy wavefront needs on its
// way to the source load: they sit together so that they arrive in one batch of scalar loads.
struct WalkArgs {
    const u32x4* x;             // [T][row_bytes / 16]
    u32x4* recv_x;              // [C][row_bytes / 16]
    const int64_t* slot_order;  // [entries]
    uint32_t entries;
    uint32_t source_limit;  // T*K
    uint32_t out_rows;
    uint32_t copy_per_xcd;  // workgroups of the walk one XCD takes
    uint32_t row_bytes;
    uint32_t topk_magic;  // fast divisor by K
    uint32_t topk_shift;
    uint32_t xcd_count;
    uint32_t xcd_magic;  // fast divisor by the XCD count
    uint32_t xcd_shift;
    uint32_t rows_per_block;  // list entries a workgroup (rows of up to four pieces; with packed rows: wavefronts x entries a wavefront)
    uint32_t weight_lane;     // 0: the first lane of a row moves the entry's weight; ~0: there are no weights
    const float* weights;     // [T][K] or null
    float* recv_weights;      // [C] or null
    // window-wise prefetch
    uint32_t segment_blocks;   // prefetch + copy workgroups of a segment
    uint32_t segment_magic;    // fast divisor by segment_blocks
    uint32_t segment_shift;
    uint32_t prefetch_blocks;  // prefetch workgroups at the head of a segment
    uint32_t segment_entries;  // list entries of a segment: ceil(entries / windows)
    // entry count on the device (the last of the 128 bytes a copy wavefront waits for before its list
    // entry: one more cache line of arguments on that way costs the walk a microsecond)
    uint32_t windows;  // segments of the walk
    uint32_t windows_magic;  // fast divisor by it
    uint32_t windows_shift;
    const int64_t* live_count;
    // what only a few wavefronts need: a second turn, the prefetch workgroups, the plain list walk
    uint32_t window_vectors;        // 16-byte vectors of one window's source rows
    uint32_t source_vectors;        // ... of all source rows
    uint32_t rows_magic;  // fast divisor by rows_per_block
    uint32_t rows_shift;
    // gap rows
    const int64_t* expert_counts;
    const int64_t* expert_offsets;
    uint32_t pad_blocks;
    uint32_t pad_per_xcd;
    uint32_t pad_per_expert;
    uint32_t pad_groups_per_expert;
    uint32_t row_vectors;
};
static_assert(offsetof(WalkArgs, live_count) + sizeof(const int64_t*) == 128, "what a copy wavefront waits for fits two cache lines");

// What a workgroup of the walk's grid does when it has no copy work: every XCD's copy workgroups are
// followed by its share of the workgroups that clear the alignment gaps, each wavefront one whole
// gap row (and its weight): workgroup (e, g) owns gap candidates j = g * waves .. of expert e, row
// offsets[e] + counts[e] + j while that is below offsets[e+1].
__device__ __forceinline__ void walk_gap_rows(const WalkArgs& a, uint32_t xcd, uint32_t pad_index) {
    const uint32_t pad_block = xcd * a.pad_per_xcd + pad_index;
    if (pad_index >= a.pad_per_xcd || pad_block >= a.pad_blocks)
        return;
    const uint32_t waves = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t expert = pad_block / a.pad_groups_per_expert;
    const uint32_t group = pad_block - expert * a.pad_groups_per_expert;
    const uint32_t j = group * waves + wave;
    if (j >= a.pad_per_expert)
        return;
    const int64_t out_row = uniform_load(a.expert_offsets + expert) + uniform_load(a.expert_counts + expert) + j;
    if (out_row < 0 || out_row >= uniform_load(a.expert_offsets + expert + 1) || out_row >= static_cast<int64_t>(a.out_rows))
        return;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    u32x4* dst = a.recv_x + out_row * a.row_vectors;
    for (uint32_t vector = lane; vector < a.row_vectors; vector += kWave)
        store_vec<true>(dst + vector, zero);
    if (lane == 0 && a.recv_weights != nullptr)
        a.recv_weights[out_row] = 0.0f;
}

// Window-wise source prefetch: the list is cut into segments of about one window's entries, and the
// copy workgroups of every segment are preceded by a few workgroups that read the window's source
// rows front to back (kPrefetchLoads KiB a wavefront, the data dropped).  The window's first touches
// then reach HBM as one sequential burst ahead of the segment's stores instead of one row at a time
// among them, and the copy wavefronts find their rows in the XCD's L2 (unless the write stream has
// pushed a row out again before its last use: a window close to the size of the L2 re-reads part of
// itself).  What it costs otherwise is one more L2 read per source row.
constexpr int kPrefetchLoads = 4;

// A uniform value as the compiler's vector value: what is computed from it runs on the vector unit.
__device__ __forceinline__ uint32_t vector_copy(uint32_t uniform) {
    uint32_t value;
    asm("v_mov_b32 %0, %1" : "=v"(value) : "s"(uniform));
    return value;
}

// One wavefront's copy: list entry `candidate`, the piece of its row that starts at 16-byte vector
// `lane_vector` of this lane.
template <int kSpan>
__device__ __forceinline__ void walk_copy_entry(const WalkArgs& a, uint32_t entries, uint32_t candidate, uint32_t lane_vector) {
    if (candidate >= entries)
        return;
    const int64_t entry = uniform_load_at(a.slot_order, candidate);
    const uint32_t source = static_cast<uint32_t>(entry);
    const uint32_t out_row = static_cast<uint32_t>(static_cast<uint64_t>(entry) >> 32);
    // (a negative entry has an impossible row; the empty statement keeps the two tests two
    // compare-and-branch pairs: merged into one condition they cost three more scalar instructions)
    if (out_row >= a.out_rows)
        return;
    asm volatile("");
    if (source >= a.source_limit)
        return;
    // From here on the arithmetic is the vector unit's: the scalar unit is shared by all wavefronts of
    // a compute unit and is what these short wavefronts queue for.
    const uint32_t source_v = vector_copy(source), out_row_v = vector_copy(out_row);
    const uint32_t token = fast_divide(source_v, a.topk_magic, a.topk_shift);
    const uint32_t lane_bytes = lane_vector * 16u;
    const char* from = reinterpret_cast<const char*>(a.x) + static_cast<uint64_t>(token) * a.row_bytes;
    char* to = reinterpret_cast<char*>(a.recv_x) + static_cast<uint64_t>(out_row_v) * a.row_bytes;
    u32x4 data[kSpan];
#pragma unroll
    for (int s = 0; s < kSpan; ++s) {
        const uint32_t at_bytes = lane_bytes + s * (kWave * 16u);
        // lanes past the end of the row re-read its start instead of branching around the load
        data[s] = *reinterpret_cast<const u32x4*>(from + (at_bytes < a.row_bytes ? at_bytes : 0u));
    }
    // the entry's weight rides with the first lane of its row while the payload is in flight
    // (weight_lane is no lane at all when there are no weights to move)
    if (lane_vector == a.weight_lane)
        a.recv_weights[out_row_v] = a.weights[source_v];
#pragma unroll
    for (int s = 0; s < kSpan; ++s) {
        const uint32_t at_bytes = lane_bytes + s * (kWave * 16u);
        if (at_bytes < a.row_bytes)
            store_vec<true>(reinterpret_cast<u32x4*>(to + at_bytes), data[s]);
    }
}

// The same for rows of at most 512 bytes: a wavefront moves kPack list entries at once, its lanes
// split into kPack groups of 64 / kPack that move kLaneVectors 16-byte vectors a lane, so that no
// half of it idles and there are fewer wavefronts to start.  Entry, range checks and addresses are
// per lane here (the groups of a wavefront differ in them); `candidate` is the lane's list entry
// and `vector` the first 16-byte vector of the row it moves.
template <int kPack, int kLaneVectors>
__device__ __forceinline__ void walk_copy_packed(const WalkArgs& a, uint32_t entries, uint32_t candidate, uint32_t vector) {
    if (candidate >= entries)
        return;
    const int64_t entry = a.slot_order[candidate];
    const uint32_t source = static_cast<uint32_t>(entry);
    const uint32_t out_row = static_cast<uint32_t>(static_cast<uint64_t>(entry) >> 32);
    // (a negative entry has an impossible row)
    if (out_row >= a.out_rows || source >= a.source_limit || vector * 16u >= a.row_bytes)
        return;
    const uint32_t token = fast_divide(source, a.topk_magic, a.topk_shift);
    const char* from = reinterpret_cast<const char*>(a.x) + static_cast<uint64_t>(token) * a.row_bytes;
    char* to = reinterpret_cast<char*>(a.recv_x) + static_cast<uint64_t>(out_row) * a.row_bytes;
    constexpr uint32_t kStride = (kWave / kPack) * 16u;
    u32x4 data[kLaneVectors];
#pragma unroll
    for (int s = 0; s < kLaneVectors; ++s) {
        const uint32_t at_bytes = vector * 16u + s * kStride;
        data[s] = *reinterpret_cast<const u32x4*>(from + (at_bytes < a.row_bytes ? at_bytes : 0u));
    }
    if (vector == a.weight_lane)
        a.recv_weights[out_row] = a.weights[source];
#pragma unroll
    for (int s = 0; s < kLaneVectors; ++s) {
        const uint32_t at_bytes = vector * 16u + s * kStride;
        if (at_bytes < a.row_bytes)
            store_vec<true>(reinterpret_cast<u32x4*>(to + at_bytes), data[s]);
    }
}

// The list's live entry count from the word the layout stored: a word that cannot be a count
// (negative, or above `limit`) counts as zero.  Two 32-bit scalar tests; the 64-bit comparisons go
// through the vector unit.
__device__ __forceinline__ uint32_t live_entries(int64_t word, uint32_t limit) {
    uint32_t high = static_cast<uint32_t>(static_cast<uint64_t>(word) >> 32);
    asm volatile("" : "+s"(high));  // (keeps the compiler from fusing the two tests into a 64-bit one)
    const uint32_t low = high != 0 ? 0xffffffffu : static_cast<uint32_t>(word);
    return low <= limit ? low : 0u;
}

// One workgroup's turn at the slot-order walk; `block` is its position in the walk.
// Without prefetch the walk is the list front to back, rows_per_block entries a workgroup.
// With prefetch the walk is cut into one segment per window of the list: `prefetch_blocks`
// workgroups that read the window's source rows, then `segment_blocks - prefetch_blocks`
// workgroups that copy the segment's share of the list, entries [s * segment_entries, (s + 1) *
// segment_entries) of it.  The windows hold nearly the same number of entries each, so equal shares
// follow them closely (a skewed mask only costs locality).  With the entry count on the device the
// host sizes the segments' workgroups for the count it expects and the share follows the live count:
// workgroups beyond it leave at once, and where it is larger they take more than one turn.
template <int kPieces, int kSpan, bool kDeviceCount, bool kPrefetch>
__device__ __forceinline__ void walk_copy(const WalkArgs& a, uint32_t entries, uint32_t segment_entries, uint32_t block) {
    // kPieces -4 / -8: rows of at most 512 / 256 bytes, four / eight entries a wavefront, kSpan vectors a lane
    constexpr int kPack = kPieces < 0 ? -kPieces : 1;
    constexpr int kRowPieces = kPieces < 0 ? 1 : kPieces;
    // the entry of this lane within its workgroup and the first 16-byte vector of the row it moves
    uint32_t in_block = 0, lane_vector;
    if (kPieces == 0) {
        lane_vector = kSpan == 1 ? threadIdx.x : (threadIdx.x / kWave) * (kSpan * kWave) + threadIdx.x % kWave;
    } else if (kPack == 1) {
        const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
        in_block = wave / kRowPieces;
        lane_vector = kSpan == 1 ? threadIdx.x - in_block * (kRowPieces * kWave)
                                 : (wave - in_block * kRowPieces) * (kSpan * kWave) + threadIdx.x % kWave;
    } else {
        in_block = threadIdx.x / (kWave / kPack);
        lane_vector = threadIdx.x % (kWave / kPack);
    }
    if (!kPrefetch) {
        const uint32_t candidate = kPieces == 0 ? block : block * a.rows_per_block + in_block;
        if (kPack == 1)
            walk_copy_entry<kSpan>(a, entries, candidate, lane_vector);
        else
            walk_copy_packed<kPack, kSpan>(a, entries, candidate, lane_vector);
        return;
    }
    const uint32_t segment = fast_divide(block, a.segment_magic, a.segment_shift);
    const uint32_t within = block - segment * a.segment_blocks;
    if (within < a.prefetch_blocks) {
        const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
        const uint32_t waves = blockDim.x / kWave;
        const uint64_t window_first = static_cast<uint64_t>(segment) * a.window_vectors;
        uint64_t window_end = window_first + a.window_vectors;
        if (window_end > a.source_vectors)
            window_end = a.source_vectors;
        const uint64_t first = window_first + static_cast<uint64_t>(within * waves + wave) * (kPrefetchLoads * kWave);
        if (first < window_end) {
            u32x4 fetched[kPrefetchLoads];
#pragma unroll
            for (int u = 0; u < kPrefetchLoads; ++u) {
                const uint64_t from = first + u * kWave + threadIdx.x % kWave;
                fetched[u] = a.x[from < window_end ? from : window_first];
            }
#pragma unroll
            for (int u = 0; u < kPrefetchLoads; ++u)
                asm volatile("" ::"v"(fetched[u].x), "v"(fetched[u].y), "v"(fetched[u].z), "v"(fetched[u].w));
        }
        __builtin_amdgcn_endpgm();
    }
    const uint32_t copy_block = within - a.prefetch_blocks;
    uint32_t in_segment = kPieces == 0 ? copy_block : copy_block * a.rows_per_block + in_block;
    const uint32_t segment_first = segment * segment_entries;
    if (!kDeviceCount) {
        if (in_segment < segment_entries) {
            if (kPack == 1)
                walk_copy_entry<kSpan>(a, entries, segment_first + in_segment, lane_vector);
            else
                walk_copy_packed<kPack, kSpan>(a, entries, segment_first + in_segment, lane_vector);
        }
        return;
    }
    // the first turn stands alone: a second one is the exception (a live count above what the grid
    // was sized for), and a loop around both makes every wavefront pay for what only a loop needs
    if (in_segment >= segment_entries)
        return;
    if (kPack == 1)
        walk_copy_entry<kSpan>(a, entries, segment_first + in_segment, lane_vector);
    else
        walk_copy_packed<kPack, kSpan>(a, entries, segment_first + in_segment, lane_vector);
    // (list entries the copy workgroups of a segment cover in one turn)
    const uint32_t turn_entries = (a.segment_blocks - a.prefetch_blocks) * a.rows_per_block;
    in_segment += turn_entries;
    if (__builtin_expect(in_segment < segment_entries, 0)) {
        do {
            if (kPack == 1)
                walk_copy_entry<kSpan>(a, entries, segment_first + in_segment, lane_vector);
            else
                walk_copy_packed<kPack, kSpan>(a, entries, segment_first + in_segment, lane_vector);
            in_segment += turn_entries;
        } while (in_segment < segment_entries);
    }
}

// The slot-order walk.  Its wavefronts are short (a list entry, a source load, a store) and there are
// hundreds of thousands of them, so the scalar instructions each one spends on finding its work are a
// throughput limit of their own (a compute unit issues one a cycle): everything on the way to the
// load is kept to the minimum, and the gap rows live behind the one test that ends a wavefront with
// no copy work.
//   kPieces 0 : one workgroup a list entry, one wavefront a piece of the row (rows of 5 to 16 pieces)
//   kPieces 1..4 : rows of that many pieces, rows_per_block entries a workgroup
//   kPieces -4, -8 : rows of up to 512 / 256 bytes, four / eight entries a wavefront
//   kSpan   : 1 KiB chunks a wavefront moves (a piece); with packed rows, 16-byte vectors a lane moves
template <int kPieces, int kSpan, bool kDeviceCount, bool kPrefetch>
__global__ void __launch_bounds__(1024) dispatch_walk_kernel(const WalkArgs a) {
    NANOEP_FETCH_ARGS_4(a.x, a.recv_x, a.slot_order, a.entries);
    NANOEP_FETCH_ARGS_4(a.source_limit, a.out_rows, a.copy_per_xcd, a.row_bytes);
    NANOEP_FETCH_ARGS_4(a.topk_magic, a.topk_shift, a.xcd_count, a.xcd_magic);
    NANOEP_FETCH_ARGS_4(a.xcd_shift, a.rows_per_block, a.weight_lane, a.weights);
    NANOEP_FETCH_ARGS_2(a.recv_weights, a.weights);
    if (kPrefetch) {
        NANOEP_FETCH_ARGS_4(a.segment_blocks, a.segment_magic, a.segment_shift, a.prefetch_blocks);
        NANOEP_FETCH_ARGS_2(a.segment_entries, a.segment_entries);
    }
    // the live count's load is on every copy wavefront's way to its list entry: it leaves with the
    // first batch of arguments and is in flight during the index arithmetic below
    int64_t live = 0;
    uint32_t block = blockIdx.x;
    if (kDeviceCount) {
        NANOEP_FETCH_ARGS_4(a.windows, a.windows_magic, a.windows_shift, a.live_count);
        live = uniform_load_begin(a.live_count, block);
    }
    const uint32_t index_in_xcd = fast_divide(block, a.xcd_magic, a.xcd_shift);
    const uint32_t xcd = block - index_in_xcd * a.xcd_count;
    if (!kDeviceCount || kPrefetch) {
        // the grid's shape is the host's: with prefetch the segments are the windows of the batch
        if (index_in_xcd >= a.copy_per_xcd) {
            walk_gap_rows(a, xcd, index_in_xcd - a.copy_per_xcd);
            __builtin_amdgcn_endpgm();
        }
        uint32_t entries = a.entries, segment_entries = a.segment_entries;
        if (kDeviceCount) {
            // a word that cannot be a count (the layout did not run) walks nothing
            live = uniform_load_end(live);
            entries = live_entries(live, a.source_limit);
            segment_entries = fast_divide(entries + a.windows - 1, a.windows_magic, a.windows_shift);
        }
        walk_copy<kPieces, kSpan, kDeviceCount, kPrefetch>(a, entries, segment_entries, xcd * a.copy_per_xcd + index_in_xcd);
        __builtin_amdgcn_endpgm();
    }
    // The entry count is on the device and the walk is the plain list: the live list may be shorter
    // than what the grid was sized for (the rest of the grid leaves at once) or longer (workgroups
    // then take more than one turn, a grid's worth of list positions apart).  A word that cannot be a
    // count (the layout did not run) walks nothing.
    live = uniform_load_end(live);
    const uint32_t entries = live_entries(live, a.source_limit);
    const uint32_t copy_blocks = kPieces == 0 ? entries : fast_divide(entries + a.rows_per_block - 1, a.rows_magic, a.rows_shift);
    const uint32_t copy_per_xcd = fast_divide(copy_blocks + a.xcd_count - 1, a.xcd_magic, a.xcd_shift);
    const uint32_t copy_turns = copy_per_xcd > a.copy_per_xcd ? a.copy_per_xcd : copy_per_xcd;
    if (index_in_xcd < copy_turns) {
        for (uint32_t at = index_in_xcd; at < copy_per_xcd; at += a.copy_per_xcd)
            walk_copy<kPieces, kSpan, kDeviceCount, kPrefetch>(a, entries, 0u, xcd * copy_per_xcd + at);
    } else {
        walk_gap_rows(a, xcd, index_in_xcd - copy_turns);
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
    const u32x4 data = load_vec<true>(x + static_cast<uint64_t>(token) * vectors + (in_row ? vector : 0u));
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
    const int vectors = hidden / 8;
    const int row_chunks = (vectors + kWave - 1) / kWave;
    // The slot-order walk is used whenever the handle carries the list.  With cache-resident sources and
    // fewer than eight token blocks the token-order walk is up to 15 % faster, but with cold sources
    // it is 25-60 % slower at every size, so the list decides.  A wavefront moves one 1 KiB chunk; two
    // once the source outgrows the last-level cache (the single-chunk walk then loses a quarter of
    // its rate) and as many as it takes for a row to fit the 16 wavefronts of a workgroup
    // (NANOEP_DISPATCH_SPAN=1|2|4 asks for a number).  The walk addresses the list with 32-bit byte
    // offsets: list buffers of 2^29 entries and more, and rows beyond 64 KiB, take the token-order walk.
    int span = static_cast<int64_t>(num_tokens) * hidden * 2 > kLastLevelCacheBytes ? 2 : 1;
    if (tuning.dispatch_span == 1 || tuning.dispatch_span == 2 || tuning.dispatch_span == 4)
        span = tuning.dispatch_span;
    while (span < 4 && (row_chunks + span - 1) / span > kMaxWavesPerBlock)
        span *= 2;
    const int pieces = (row_chunks + span - 1) / span;
    const bool ordered = expand && slot_order != nullptr && order_bound > 0 && tuning.dispatch_order != 0 &&
                         pieces <= kMaxWavesPerBlock && order_bound < (int64_t{1} << 29);
    if (ordered && slot_order_entries > order_bound)
        return NANOEP_ERR_INVALID_ARGUMENT;
    if (num_tokens * num_topk >= (int64_t{1} << 31) || static_cast<int64_t>(num_tokens) * vectors >= (int64_t{1} << 32))
        return NANOEP_ERR_INVALID_ARGUMENT;
    auto stream = static_cast<hipStream_t>(stream_handle);
    // No expert's gap exceeds alignment-1 rows, and all gaps together stay below C.
    const int64_t pad_per_expert = !pad ? 0 : (alignment - 1 < expanded_capacity ? alignment - 1 : expanded_capacity);

    if (ordered) {
        // A negative entry count defers to the count word the layout stored behind the list.  -1 sizes the
        // grid for the most entries the list can hold (T * K), -g for about g of them: workgroups beyond
        // the live count leave at once, and where the live count is above g workgroups take several turns.
        const int64_t* live_count = slot_order_entries < 0 ? slot_order + order_bound : nullptr;
        if (live_count != nullptr) {
            const int64_t most = num_tokens * num_topk;
            const int64_t expected = slot_order_entries == -1 ? most : -slot_order_entries;
            slot_order_entries = expected < most ? expected : most;
        }
        // Rows of up to four pieces share a workgroup (kPieces of the kernel); longer rows take one each.
        // Rows of at most 512 bytes fill half a wavefront or less: the lanes of a wavefront then split
        // into four or eight groups that move one list entry each, a lane one or two 16-byte vectors of
        // it (up to 128 bytes: 8 entries x 1 vector; up to 256: 8 x 2; up to 512: 4 x 2).  Sources from
        // HBM / cache resident, one entry a wavefront -> packed: 65536 x 256 top-8 75.1 -> 58.3 us /
        // 61.3 -> 46.3; 65536 x 192 66.4 -> 46.5 / 57.6 -> 31.1; 65536 x 128 57.6 -> 33.0 / 51.8 -> 24.5;
        // 65536 x 64 top-4 31.5 -> 10.6 / 29.9 -> 8.3.  (Two entries of 32 lanes x 1 vector at 512-byte
        // rows: 64.2 / 45.5; the same split for rows of 1 KiB and more loses 3 to 10 %.)
        // NANOEP_DISPATCH_PACK=1 keeps one entry a wavefront.
        int pack = 1, lane_vectors = 1;
        if (row_chunks == 1 && vectors <= kWave / 2 && tuning.dispatch_pack != 1) {
            pack = vectors <= kWave / 4 ? 8 : 4;
            lane_vectors = vectors <= kWave / 8 ? 1 : 2;
        }
        const int walk_pieces = pack > 1 ? 1 : pieces;
        const int kernel_pieces = walk_pieces <= 4 ? walk_pieces : 0;
        int rows_per_block = 1;
        if (kernel_pieces != 0) {
            rows_per_block = tuning.rows_per_block;
            if (rows_per_block < 1 || rows_per_block * walk_pieces > kMaxWavesPerBlock)
                rows_per_block = default_walk_rows(walk_pieces);
        }
        const int64_t waves = static_cast<int64_t>(walk_pieces) * rows_per_block;
        const int64_t entries_per_block = static_cast<int64_t>(rows_per_block) * pack;
        const int64_t copy_blocks = (slot_order_entries + entries_per_block - 1) / entries_per_block;
        const int64_t pad_groups_per_expert = (pad_per_expert + waves - 1) / waves;
        const int64_t pad_blocks = num_local_experts * pad_groups_per_expert;
        // Prefetch workgroups ahead of every window's share of the list.  The list's windows hold
        // nearly the same number of entries each, so equal shares of the list follow them closely.
        // With sources that come from HBM it gains 5 to 22 % (rows of 512 elements most, 7168 least),
        // with sources that sit in the last-level cache it costs 0 to 4 %: on unless
        // NANOEP_DISPATCH_PREFETCH=0.
        const int window_tokens = nanoep_layout_block_tokens(num_tokens, num_local_experts, hidden);
        const bool prefetch = window_tokens > 0 && copy_blocks > 0 && tuning.dispatch_prefetch != 0;
        // Segments are the windows of the batch; each takes the workgroups that copy its share of the
        // entries the host expects, behind the ones that read the window's rows.
        int64_t segment_entries = 0, segment_copy_blocks = 0, segment_prefetch_blocks = 0, windows = 1;
        if (prefetch) {
            windows = (num_tokens + window_tokens - 1) / window_tokens;
            segment_entries = (slot_order_entries + windows - 1) / windows;
            segment_copy_blocks = (segment_entries + entries_per_block - 1) / entries_per_block;
            const int64_t window_kib = (static_cast<int64_t>(window_tokens) * vectors + kWave - 1) / kWave;
            segment_prefetch_blocks = (window_kib + waves * kPrefetchLoads - 1) / (waves * kPrefetchLoads);
        }
        const int64_t walk_blocks = prefetch ? windows * (segment_copy_blocks + segment_prefetch_blocks) : copy_blocks;
        if (walk_blocks + pad_blocks >= (int64_t{1} << 31) - 2 * int64_t{xcds.count})
            return NANOEP_ERR_INVALID_ARGUMENT;
        const uint32_t copy_per_xcd = static_cast<uint32_t>((walk_blocks + xcds.count - 1) / xcds.count);
        const uint32_t pad_per_xcd = static_cast<uint32_t>((pad_blocks + xcds.count - 1) / xcds.count);
        const FastDivisor topk_divisor = make_fast_divisor(static_cast<uint32_t>(num_topk));
        const FastDivisor rows_divisor = make_fast_divisor(static_cast<uint32_t>(entries_per_block));
        const FastDivisor windows_divisor = make_fast_divisor(static_cast<uint32_t>(windows));
        const FastDivisor segment_divisor =
            make_fast_divisor(static_cast<uint32_t>(prefetch ? segment_copy_blocks + segment_prefetch_blocks : 1));
        WalkArgs a{};
        a.x = static_cast<const u32x4*>(x);
        a.recv_x = static_cast<u32x4*>(recv_x);
        a.slot_order = slot_order;
        a.entries = static_cast<uint32_t>(slot_order_entries);
        a.source_limit = static_cast<uint32_t>(num_tokens * num_topk);
        a.out_rows = static_cast<uint32_t>(out_rows);
        a.copy_per_xcd = copy_per_xcd;
        a.row_bytes = static_cast<uint32_t>(vectors) * 16u;
        a.topk_magic = topk_divisor.magic;
        a.topk_shift = topk_divisor.shift;
        a.xcd_count = xcds.count;
        a.xcd_magic = xcds.magic;
        a.xcd_shift = xcds.shift;
        a.rows_per_block = static_cast<uint32_t>(entries_per_block);
        a.weight_lane = recv_weights == nullptr ? 0xffffffffu : 0u;
        a.weights = weights;
        a.recv_weights = recv_weights;
        a.segment_blocks = static_cast<uint32_t>(segment_copy_blocks + segment_prefetch_blocks);
        a.segment_magic = segment_divisor.magic;
        a.segment_shift = segment_divisor.shift;
        a.prefetch_blocks = static_cast<uint32_t>(segment_prefetch_blocks);
        a.window_vectors = static_cast<uint32_t>(static_cast<int64_t>(window_tokens) * vectors);
        a.source_vectors = static_cast<uint32_t>(num_tokens * vectors);
        a.segment_entries = static_cast<uint32_t>(segment_entries);
        a.windows = static_cast<uint32_t>(windows);
        a.windows_magic = windows_divisor.magic;
        a.windows_shift = windows_divisor.shift;
        a.rows_magic = rows_divisor.magic;
        a.rows_shift = rows_divisor.shift;
        a.live_count = live_count;
        a.expert_counts = expert_counts;
        a.expert_offsets = expert_offsets;
        a.pad_blocks = static_cast<uint32_t>(pad_blocks);
        a.pad_per_xcd = pad_per_xcd;
        a.pad_per_expert = static_cast<uint32_t>(pad_per_expert);
        a.pad_groups_per_expert = static_cast<uint32_t>(pad_groups_per_expert > 0 ? pad_groups_per_expert : 1);
        a.row_vectors = static_cast<uint32_t>(vectors);
        const dim3 grid(static_cast<unsigned>((int64_t{copy_per_xcd} + pad_per_xcd) * xcds.count));
        const dim3 threads(static_cast<unsigned>(waves * kWave));
        const bool device_count = live_count != nullptr;
#define NANOEP_LAUNCH_WALK(PIECES, SPAN)                                                       \
    do {                                                                                       \
        if (device_count && prefetch)                                                          \
            dispatch_walk_kernel<PIECES, SPAN, true, true><<<grid, threads, 0, stream>>>(a);   \
        else if (device_count)                                                                 \
            dispatch_walk_kernel<PIECES, SPAN, true, false><<<grid, threads, 0, stream>>>(a);  \
        else if (prefetch)                                                                     \
            dispatch_walk_kernel<PIECES, SPAN, false, true><<<grid, threads, 0, stream>>>(a);  \
        else                                                                                   \
            dispatch_walk_kernel<PIECES, SPAN, false, false><<<grid, threads, 0, stream>>>(a); \
    } while (0)
#define NANOEP_LAUNCH_WALK_PIECES(PIECES)  \
    do {                                   \
        if (span == 4)                     \
            NANOEP_LAUNCH_WALK(PIECES, 4); \
        else if (span == 2)                \
            NANOEP_LAUNCH_WALK(PIECES, 2); \
        else                               \
            NANOEP_LAUNCH_WALK(PIECES, 1); \
    } while (0)
        switch (pack > 1 ? -pack : kernel_pieces) {
            case -8:
                if (lane_vectors == 2)
                    NANOEP_LAUNCH_WALK(-8, 2);
                else
                    NANOEP_LAUNCH_WALK(-8, 1);
                break;
            case -4:
                NANOEP_LAUNCH_WALK(-4, 2);
                break;
            case 1:
                NANOEP_LAUNCH_WALK_PIECES(1);
                break;
            case 2:
                NANOEP_LAUNCH_WALK_PIECES(2);
                break;
            case 3:
                NANOEP_LAUNCH_WALK_PIECES(3);
                break;
            case 4:
                NANOEP_LAUNCH_WALK_PIECES(4);
                break;
            default:
                NANOEP_LAUNCH_WALK_PIECES(0);
                break;
        }
#undef NANOEP_LAUNCH_WALK_PIECES
#undef NANOEP_LAUNCH_WALK
        NANOEP_HIP_TRY(hipGetLastError());
        return NANOEP_OK;
    }

    // token-order walks and the compact row copy: workgroups of (64, chunks, rows)
    const int chunks = row_chunks;
    const RowBlocking blocking = pick_row_blocking(chunks, expand ? kTokenOrderWalk : kRowCopyWalk, tuning);
    const int64_t waves = static_cast<int64_t>(blocking.chunks_per_block) * blocking.rows_per_block;
    const int64_t copy_candidates = expand ? num_tokens * num_topk : num_tokens;
    const int64_t copy_blocks = (copy_candidates + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
    const int64_t pad_groups_per_expert = (pad_per_expert + waves - 1) / waves;
    const int64_t pad_blocks = num_local_experts * pad_groups_per_expert;
    if (copy_blocks + pad_blocks >= (int64_t{1} << 31) - 2 * int64_t{xcds.count})
        return NANOEP_ERR_INVALID_ARGUMENT;
    const uint32_t copy_per_xcd = static_cast<uint32_t>((copy_blocks + xcds.count - 1) / xcds.count);
    const uint32_t pad_per_xcd = static_cast<uint32_t>((pad_blocks + xcds.count - 1) / xcds.count);
    int topk_shift = -1;
    if ((num_topk & (num_topk - 1)) == 0)
        for (topk_shift = 0; (1 << topk_shift) < num_topk; ++topk_shift) {
        }
    const dim3 grid(static_cast<unsigned>((int64_t{copy_per_xcd} + pad_per_xcd) * xcds.count));
    const dim3 block(kWave, blocking.chunks_per_block, blocking.rows_per_block);
    const FastDivisor parts_divisor = make_fast_divisor(blocking.parts);
    if (!expand) {
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
