// Combine gather-reduce: fp32 accumulation in ascending k, bias, weight restore, compact row copy.

#include "nanoep_device.h"

namespace nanoep {
namespace {

// flags of the gather kernels
constexpr int kCombineMultipleReduction = 1;  // round sums of two or more rows to bf16 once before the final pass
constexpr int kCombineAgentStores = 2;        // agent-scope stores for the output instead of nontemporal ones
// largest output (bytes) that is written with agent-scope stores
constexpr int64_t kAgentStoreOutputBytes = int64_t{88} << 20;
// rows of a token that combine_held_kernel fetches at a time, and (token, k) pairs whose weights a
// lane of its side workgroups restores
constexpr int kHeldRows = 8;
constexpr int kHeldSideEntries = 8;

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

// Expanded layout.  One wavefront produces one 1 KiB chunk of one source token's output row.  A
// workgroup is (64, chunks_per_block, tokens_per_block).  Lane k fetches the token's k-th slot (from
// token_slots[t][k], or dst_slots[t] -> recv_metadata[row][2+k]); the slots are broadcast to
// scalars, the kGroup rows are fetched with back-to-back nontemporal 128-bit loads (a masked k
// re-reads row 0 so that the loads stay unconditional) and the valid ones are added in ascending k
// starting from +0.0f; the optional bias is added once and the sum is rounded to bf16 once.
template <int kGroup, bool kDirectSlots>
__global__ void __launch_bounds__(1024) combine_rows_kernel(const u32x4* __restrict__ y,                // [C][vectors]
                                                            const float* __restrict__ weights,         // [C] or null
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
                                                            int flags) {  // kCombineMultipleReduction | kCombineAgentStores
    NANOEP_FETCH_ARGS_4(y, weights, bias, out_x);
    NANOEP_FETCH_ARGS_4(recv_metadata, dst_slots, token_slots, out_weights);
    NANOEP_FETCH_ARGS_4(recv_count, y_rows, num_tokens, parts);
    NANOEP_FETCH_ARGS_4(parts_magic, parts_shift, chunks_per_block, tokens_per_block);
    NANOEP_FETCH_ARGS_4(vectors, chunks, num_topk, flags);
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

    // slot: expanded slot of this token's k = lane, -1 when masked
    bool received = true;
    const int32_t* slots;
    if (kDirectSlots) {
        slots = token_slots + static_cast<int64_t>(token) * num_topk;
    } else {
        const int64_t row = uniform_load(dst_slots + token);
        received = row >= 0 && row < recv_count;
        slots = recv_metadata + (received ? row : 0) * (num_topk + 2) + 2;
    }
    int slot = -1;
    if (received && lane < num_topk)
        slot = slots[lane];
    const bool valid = slot >= 0 && slot < y_rows;
    const uint64_t valid_mask = __ballot(valid);
    const int gathered = valid_mask == 0 ? 0 : num_topk;

    u32x4 bias_data = {0u, 0u, 0u, 0u};
    if (bias != nullptr)
        bias_data = load_vec<true>(bias + static_cast<int64_t>(token) * vectors + load_vector);

    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int base = 0; base < gathered; base += kGroup) {
        u32x4 data[kGroup];
#pragma unroll
        for (int k = 0; k < kGroup; ++k) {
            const bool live = (valid_mask >> (base + k)) & 1;
            int64_t source_row = 0;
            if (live)
                source_row = static_cast<int64_t>(__builtin_amdgcn_readlane(slot, (base + k) & (kWave - 1)));
            data[k] = load_vec<true>(y + source_row * vectors + load_vector);
        }
#pragma unroll
        for (int k = 0; k < kGroup; ++k)
            if ((valid_mask >> (base + k)) & 1)
                accumulate(acc, data[k]);
    }
    if ((flags & kCombineMultipleReduction) && __popcll(valid_mask) >= 2) {
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
        if (flags & kCombineAgentStores)
            store_vec_agent(out_x + static_cast<int64_t>(token) * vectors + vector, packed);
        else
            store_vec<true>(out_x + static_cast<int64_t>(token) * vectors + vector, packed);
    }

    if (chunk == 0 && out_weights != nullptr && lane < num_topk)
        out_weights[static_cast<int64_t>(token) * num_topk + lane] = valid ? weights[slot] : 0.0f;
}

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
                                                                int flags,  // kCombineMultipleReduction | kCombineAgentStores
                                                                uint32_t topk_magic,  // fast divisor by K
                                                                uint32_t topk_shift,
                                                                uint32_t side_blocks) {
    NANOEP_FETCH_ARGS_4(y, token_slots, out_x, bias);
    NANOEP_FETCH_ARGS_4(tokens, y_rows, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    NANOEP_FETCH_ARGS_4(chunks, topk, flags, out_weights);
    if (blockIdx.x < side_blocks) {
        // weights back to their (token, k): one lane each, in workgroups of their own at the front
        // of the grid (on the first payload wavefront of a row they are a second round trip)
        const uint32_t wave = threadIdx.z * chunks_per_block + threadIdx.y;
        const uint32_t flat = (blockIdx.x * (chunks_per_block * rows_per_block) + wave) * kWave + threadIdx.x;
        if (fast_divide(flat, topk_magic, topk_shift) >= tokens)
            return;
        const int32_t slot = token_slots[flat];
        out_weights[flat] = slot >= 0 && static_cast<uint32_t>(slot) < y_rows ? weights[slot] : 0.0f;
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
    if ((flags & kCombineMultipleReduction) && valid_count >= 2) {
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
        if (flags & kCombineAgentStores)
            store_vec_agent(out_x + static_cast<uint64_t>(token) * vectors + vector, packed);
        else
            store_vec<true>(out_x + static_cast<uint64_t>(token) * vectors + vector, packed);
    }
}

// Expanded layout with the slot table at hand and five or more rows a token: one wavefront (a
// workgroup of its own) produces the same 1 KiB chunk of the output rows of up to kUnits tokens
// and holds the packed sums back in registers until the last one is done.  The units are
// sized so that all wavefronts of the launch are resident at once wherever the batch allows it: the
// whole device then reads first and writes last, and HBM sees the output as one burst behind the
// gather instead of a write among every eight reads.  A token's rows are fetched eight at a time (a
// masked k re-reads row 0 so that the loads stay unconditional).
template <int kUnits>
__global__ void __launch_bounds__(kWave) combine_held_kernel(const u32x4* __restrict__ y,              // [C][vectors]
                                                             const float* __restrict__ weights,       // [C] or null
                                                             const u32x4* __restrict__ bias,          // [T][vectors] or null
                                                             const int32_t* __restrict__ token_slots,  // [T][K]
                                                             u32x4* __restrict__ out_x,               // [T][vectors]
                                                             float* __restrict__ out_weights,         // [T][K] or null
                                                             uint32_t tokens,
                                                             uint32_t y_rows,
                                                             uint32_t chunks,
                                                             uint32_t chunks_magic,  // fast divisor by chunks
                                                             uint32_t chunks_shift,
                                                             uint32_t vectors,
                                                             uint32_t topk,
                                                             int flags,  // kCombineMultipleReduction | kCombineAgentStores
                                                             uint32_t side_blocks,
                                                             uint32_t units,        // tokens a wavefront, at most kUnits
                                                             uint32_t first_scale,  // first token of a wavefront = group * first_scale
                                                             uint32_t stride) {     // distance between a wavefront's tokens
    NANOEP_FETCH_ARGS_4(y, token_slots, out_x, bias);
    NANOEP_FETCH_ARGS_4(tokens, y_rows, chunks, chunks_magic);
    NANOEP_FETCH_ARGS_4(chunks_shift, vectors, topk, flags);
    NANOEP_FETCH_ARGS_4(side_blocks, units, first_scale, stride);
    const uint32_t lane = threadIdx.x;
    if (blockIdx.x < side_blocks) {
        // weights back to their (token, k): kHeldSideEntries consecutive ones a lane, in workgroups
        // of their own at the front of the grid (on a payload wavefront they are one more round
        // trip); few enough wavefronts to count little against what the launch is sized for
        const uint32_t pairs = tokens * topk;
        const uint32_t flat = (blockIdx.x * kWave + lane) * kHeldSideEntries;
        int32_t slot[kHeldSideEntries];
#pragma unroll
        for (int j = 0; j < kHeldSideEntries; ++j)
            slot[j] = flat + j < pairs ? token_slots[flat + j] : -1;
        float restored[kHeldSideEntries];
#pragma unroll
        for (int j = 0; j < kHeldSideEntries; ++j)
            restored[j] = slot[j] >= 0 && static_cast<uint32_t>(slot[j]) < y_rows ? weights[slot[j]] : 0.0f;
#pragma unroll
        for (int j = 0; j < kHeldSideEntries; ++j)
            if (flat + j < pairs)
                out_weights[flat + j] = restored[j];
        return;
    }
    const uint32_t payload_block = blockIdx.x - side_blocks;
    const uint32_t group = fast_divide(payload_block, chunks_magic, chunks_shift);
    const uint32_t chunk = payload_block - group * chunks;
    const uint32_t vector = chunk * kWave + lane;
    const bool in_row = vector < vectors;
    // lanes past the end of a short row re-read vector 0 instead of branching around the loads
    const uint32_t load_vector = in_row ? vector : 0u;
    // this wavefront's tokens: first, first + stride, ... (`units` of them while they are tokens).
    // Consecutive tokens (first = group * units, stride 1), or, when the whole launch is resident at
    // once, every groups-th token (first = group, stride = groups): the tokens in flight at any
    // moment are then neighbours, and so are the rows they read in every expert's segment.
    const uint32_t first = group * first_scale;
    u32x4 packed[kUnits];
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
        const uint32_t token = first + static_cast<uint32_t>(u) * stride;
        if (static_cast<uint32_t>(u) >= units || token >= tokens)
            continue;
        // lane k fetches the token's k-th slot; the slots are broadcast to scalars below
        int slot = -1;
        if (lane < topk)
            slot = token_slots[static_cast<uint64_t>(token) * topk + lane];
        const bool valid = slot >= 0 && static_cast<uint32_t>(slot) < y_rows;
        const uint32_t valid_mask = static_cast<uint32_t>(__ballot(valid));
        u32x4 bias_data = {0u, 0u, 0u, 0u};
        if (bias != nullptr)
            bias_data = load_vec<true>(bias + static_cast<uint64_t>(token) * vectors + load_vector);
        float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        // eight rows a pass, in ascending k
        for (uint32_t base = 0; base < (valid_mask != 0 ? topk : 0u); base += kHeldRows) {
            u32x4 data[kHeldRows];
#pragma unroll
            for (int k = 0; k < kHeldRows; ++k) {
                uint64_t source_row = 0;
                if ((valid_mask >> (base + k)) & 1)
                    source_row = static_cast<uint32_t>(__builtin_amdgcn_readlane(slot, (base + k) & (kWave - 1)));
                data[k] = load_vec<true>(y + source_row * vectors + load_vector);
            }
#pragma unroll
            for (int k = 0; k < kHeldRows; ++k)
                if ((valid_mask >> (base + k)) & 1)
                    accumulate(acc, data[k]);
        }
        if ((flags & kCombineMultipleReduction) && __popc(valid_mask) >= 2) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                acc[j] = 0.0f + __uint_as_float(bf16_round(acc[j]) << 16);
        }
        if (bias != nullptr)
            accumulate(acc, bias_data);
        packed[u].x = bf16_round(acc[0]) | (bf16_round(acc[1]) << 16);
        packed[u].y = bf16_round(acc[2]) | (bf16_round(acc[3]) << 16);
        packed[u].z = bf16_round(acc[4]) | (bf16_round(acc[5]) << 16);
        packed[u].w = bf16_round(acc[6]) | (bf16_round(acc[7]) << 16);
        // the packed row is pinned here: left to itself the compiler keeps every token's eight fp32 sums
        // and rounds them all at the end, which doubles the registers held and costs the compute units
        // a quarter of their resident wavefronts
        asm volatile("" : "+v"(packed[u].x), "+v"(packed[u].y), "+v"(packed[u].z), "+v"(packed[u].w)::"memory");
    }
    if (!in_row)
        return;
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
        const uint32_t token = first + static_cast<uint32_t>(u) * stride;
        if (static_cast<uint32_t>(u) < units && token < tokens) {
            u32x4* to = out_x + static_cast<uint64_t>(token) * vectors + vector;
            if (flags & kCombineAgentStores)
                store_vec_agent(to, packed[u]);
            else
                store_vec<true>(to, packed[u]);
        }
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
                                                               uint32_t topk,
                                                               uint32_t topk_magic,  // fast divisor by K
                                                               uint32_t topk_shift,
                                                               uint32_t side_blocks) {
    NANOEP_FETCH_ARGS_4(y, dst_slots, out_x, bias);
    NANOEP_FETCH_ARGS_4(tokens, recv_count, parts, parts_magic);
    NANOEP_FETCH_ARGS_4(parts_shift, chunks_per_block, rows_per_block, vectors);
    if (blockIdx.x < side_blocks) {
        // weights back to their (token, k), zero for masked choices and tokens that were not sent: one
        // lane each, in workgroups of their own at the front of the grid.  On the first payload wavefront
        // of every row the two dependent lookups cost 22 us of 104 at 32768 x 4096, top-8.
        const uint32_t wave = threadIdx.z * chunks_per_block + threadIdx.y;
        const uint32_t flat = (blockIdx.x * (chunks_per_block * rows_per_block) + wave) * kWave + threadIdx.x;
        const uint32_t token = fast_divide(flat, topk_magic, topk_shift);
        if (token >= tokens)
            return;
        const uint32_t k = flat - token * topk;
        const int64_t row = dst_slots[token];
        float weight = 0.0f;
        if (row >= 0 && row < static_cast<int64_t>(recv_count) && recv_metadata[row * (topk + 2) + 2 + k] >= 0)
            weight = weights[row * topk + k];
        out_weights[flat] = weight;
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
}

// Wavefronts of combine_held_kernel<kUnits> that one compute unit holds at once: four SIMDs, each with
// 512 vector registers a lane shared by its wavefronts (granules of 8), at most 8 wavefronts a SIMD.
// The register count is the compiler's, so the runtime is asked for it; `fallback` (what this file
// was written against) is the answer when the runtime gives none.
template <int kUnits>
int held_wavefronts_per_cu(int fallback) {
    hipFuncAttributes attributes{};
    if (hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&combine_held_kernel<kUnits>)) != hipSuccess ||
        attributes.numRegs <= 0) {
        (void)hipGetLastError();
        return fallback;
    }
    const int granules = (attributes.numRegs + 7) / 8 * 8;
    const int per_simd = 512 / granules;
    return 4 * (per_simd > 8 ? 8 : per_simd < 1 ? 1 : per_simd);
}

}  // namespace

void held_combine_residency(int out[4]) {
    out[0] = held_wavefronts_per_cu<2>(out[0]);
    out[1] = held_wavefronts_per_cu<4>(out[1]);
    out[2] = held_wavefronts_per_cu<8>(out[2]);
    out[3] = held_wavefronts_per_cu<16>(out[3]);
}

}  // namespace nanoep

using namespace nanoep;

extern "C" {

int nanoep_combine(const void* y, const float* weights, const void* bias, const int32_t* recv_metadata,
                   const int64_t* dst_slots, const int32_t* token_slots, int64_t recv_count, int64_t y_rows,
                   int64_t num_tokens, int hidden, int num_topk, int expand, int multiple_reduction, void* out_x,
                   float* out_weights, int num_cus, void* stream_handle) {
    const Tuning tuning = current_tuning();
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
    const int budget_status = validate_cu_budget(num_cus, current_topology(tuning));
    if (budget_status != NANOEP_OK)
        return budget_status;
    if (num_tokens == 0)
        return NANOEP_OK;
    if (out_x == nullptr || dst_slots == nullptr || (recv_count > 0 && (recv_metadata == nullptr || y == nullptr)))
        return NANOEP_ERR_INVALID_ARGUMENT;

    const int vectors = hidden / 8;
    const int chunks = (vectors + kWave - 1) / kWave;
    // top-1 expanded combines are row copies like the compact ones
    const RowBlocking blocking = pick_row_blocking(chunks, expand && num_topk > 1 ? kTokenOrderWalk : kRowCopyWalk, tuning);
    const int64_t blocks = (num_tokens + blocking.rows_per_block - 1) / blocking.rows_per_block * blocking.parts;
    if (blocks >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const dim3 grid(static_cast<unsigned>(blocks));
    const dim3 block(kWave, blocking.chunks_per_block, blocking.rows_per_block);
    // workgroups of their own, one lane per (token, k), for the kernels that restore weights that way
    const int64_t waves = static_cast<int64_t>(blocking.chunks_per_block) * blocking.rows_per_block;
    const int64_t side_lanes = out_weights != nullptr ? num_tokens * num_topk : 0;
    const int64_t side_blocks = (side_lanes + kWave * waves - 1) / (kWave * waves);
    if (side_lanes >= (int64_t{1} << 31) || blocks + side_blocks >= (int64_t{1} << 31))
        return NANOEP_ERR_INVALID_ARGUMENT;
    const dim3 grid_with_side(static_cast<unsigned>(blocks + side_blocks));
    const FastDivisor topk_divisor = make_fast_divisor(static_cast<uint32_t>(num_topk));
    auto stream = static_cast<hipStream_t>(stream_handle);
    // the slot table only helps the expanded layout, and only when something was received
    const bool direct = token_slots != nullptr && expand && recv_count > 0;
    const FastDivisor parts_divisor = make_fast_divisor(blocking.parts);
    // Output rows are written once among many reads.  With agent-scope stores instead of nontemporal
    // ones the gather kernels are 2 to 7 % faster while the output is small next to the last-level
    // cache (4096 x 7168 top-8: 79.9 -> 78.0 us, 4096 x 4096 top-2: 18.4 -> 17.2 us; outputs of
    // 28 to 84 MiB: 1.5 to 7 % faster) and 1 to 4 % slower from 96 MiB on.  The plain row copy of the
    // compact layout keeps the nontemporal store.  NANOEP_COMBINE_STORES=0|1 overrides.
    const bool agent_stores = tuning.combine_stores < 0 ? static_cast<int64_t>(num_tokens) * hidden * 2 <= kAgentStoreOutputBytes
                                                        : tuning.combine_stores != 0;
    const int flags = (multiple_reduction ? kCombineMultipleReduction : 0) | (agent_stores ? kCombineAgentStores : 0);
    if (!expand) {
        // y may be a null pointer when nothing was received: every token then takes the hole path
        combine_compact_kernel<<<grid_with_side, block, 0, stream>>>(
            static_cast<const u32x4*>(recv_count > 0 ? y : out_x), weights, static_cast<const u32x4*>(bias), recv_metadata,
            dst_slots, static_cast<u32x4*>(out_x), out_weights, static_cast<uint32_t>(num_tokens),
            static_cast<uint32_t>(recv_count), blocking.parts, parts_divisor.magic, parts_divisor.shift,
            blocking.chunks_per_block, blocking.rows_per_block, static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks),
            static_cast<uint32_t>(num_topk), topk_divisor.magic, topk_divisor.shift, static_cast<uint32_t>(side_blocks));
        NANOEP_HIP_TRY(hipGetLastError());
        return NANOEP_OK;
    }
    // Five or more rows a token with the slot table at hand: wavefronts that hold the sums of 2 to 16
    // tokens back and write them at their end; as many tokens a wavefront as it takes for the launch to
    // fit what the device holds at once with the registers of sixteen held rows (16 wavefronts a
    // compute unit), or a whole multiple of that when sixteen tokens a wavefront are not enough: a
    // launch a little larger than what is resident waits for its last few wavefronts with the device
    // idle (5120 x 7168 top-8 with sixteen tokens a wavefront: 104.7 us against 95.7 with one and 93.1
    // with nine; 4096 x 7168 with fourteen, six wavefronts too many: 78.8 against 74.1 with fifteen).  Against one
    // (token, chunk) a wavefront, sources from HBM: 4096 x 7168 top-8 78.2 -> 73.7 us, 8192 x 2048
    // 49.1 -> 47.6, 2048 x 7168 39.9 -> 37.8, 32768 x 1024 89.0 -> 83.4, 32768 x 512 46.1 -> 44.7,
    // 8192 x 7168 159.2 -> 155.4; 4096 x 4096 top-16 82.9 -> 79.7, 2048 x 7168 top-12 57.8 -> 55.3.  With
    // two to four rows a token the held sums lose to
    // combine_few_rows_kernel (4096 x 4096 top-2: 17.3 us against 18.1 to 30.5).
    // NANOEP_COMBINE_UNITS=1 keeps one token a wavefront, 2..16 asks for that many.
    int held_units = 0;
    int64_t held_resident = 0, held_side = 0;
    if (direct && num_topk > 4 && num_topk <= 32 && tuning.combine_units != 1) {
        // (the wavefronts of sixteen held rows a compute unit holds, on the compute units this call may use)
        const Topology topology = current_topology(tuning);
        const int64_t cus = num_cus > 0 ? num_cus : topology.cus;
        const int64_t resident = cus * topology.held_wavefronts[3];
        held_resident = resident;
        // (the side wavefronts that restore the weights are in the launch too)
        held_side = (side_lanes + kWave * kHeldSideEntries - 1) / (kWave * kHeldSideEntries);
        const int64_t work = num_tokens * chunks;
        const int64_t rounds = (work + held_side + 16 * resident - 1) / (16 * resident);
        held_units = 16;
        for (int units = 2; units <= 16; ++units) {
            // (with the registers of at most eight / four held rows a compute unit holds more wavefronts)
            const int64_t room = cus * topology.held_wavefronts[units > 8 ? 3 : units > 4 ? 2 : units > 2 ? 1 : 0];
            const int64_t payload = (num_tokens + units - 1) / units * chunks;
            if (payload <= rounds * resident && payload + held_side <= rounds * room) {
                held_units = units;
                break;
            }
        }
        if (tuning.combine_units >= 2 && tuning.combine_units <= 16)
            held_units = tuning.combine_units;
    }
    if (held_units > 0) {
        const FastDivisor chunks_divisor = make_fast_divisor(static_cast<uint32_t>(chunks));
        const int64_t held_side_blocks = held_side;
        const int64_t held_groups = (num_tokens + held_units - 1) / held_units;
        const int64_t held_blocks = held_groups * chunks + held_side_blocks;
        // A launch that is resident as a whole gives a wavefront every held_groups-th token instead of
        // consecutive ones (4096 x 7168 top-8 74.8 -> 73.6 us, 8192 x 2048 47.4 -> 46.9, 32768 x 512
        // 44.7 -> 43.5, 32768 x 1024 84.2 -> 83.7; within half a percent at 2048 x 7168, 3000 x 7168,
        // 4096 x 4096 top-16).  Launches of several rounds lose with it (16384 x 7168: 311 -> 323 us).
        const bool strided = held_groups * chunks <= held_resident;
        if (held_blocks >= (int64_t{1} << 31))
            return NANOEP_ERR_INVALID_ARGUMENT;
#define NANOEP_LAUNCH_HELD(UNITS)                                                                                      \
    combine_held_kernel<UNITS><<<dim3(static_cast<unsigned>(held_blocks)), dim3(kWave), 0, stream>>>(                 \
        static_cast<const u32x4*>(y), weights, static_cast<const u32x4*>(bias), token_slots, static_cast<u32x4*>(out_x), \
        out_weights, static_cast<uint32_t>(num_tokens), static_cast<uint32_t>(y_rows), static_cast<uint32_t>(chunks),   \
        chunks_divisor.magic, chunks_divisor.shift, static_cast<uint32_t>(vectors), static_cast<uint32_t>(num_topk), flags, \
        static_cast<uint32_t>(held_side_blocks), static_cast<uint32_t>(held_units),                                      \
        strided ? 1u : static_cast<uint32_t>(held_units), strided ? static_cast<uint32_t>(held_groups) : 1u)
        if (held_units > 8)
            NANOEP_LAUNCH_HELD(16);
        else if (held_units > 4)
            NANOEP_LAUNCH_HELD(8);
        else if (held_units > 2)
            NANOEP_LAUNCH_HELD(4);
        else
            NANOEP_LAUNCH_HELD(2);
#undef NANOEP_LAUNCH_HELD
        NANOEP_HIP_TRY(hipGetLastError());
        return NANOEP_OK;
    }
    if (direct && num_topk <= 4) {
#define NANOEP_LAUNCH_FEW(TOPK)                                                                                       \
    combine_few_rows_kernel<TOPK><<<grid_with_side, block, 0, stream>>>(                                             \
        static_cast<const u32x4*>(y), weights, static_cast<const u32x4*>(bias), token_slots,                         \
        static_cast<u32x4*>(out_x), out_weights, static_cast<uint32_t>(num_tokens), static_cast<uint32_t>(y_rows),   \
        blocking.parts, parts_divisor.magic, parts_divisor.shift, blocking.chunks_per_block, blocking.rows_per_block, \
        static_cast<uint32_t>(vectors), static_cast<uint32_t>(chunks), static_cast<uint32_t>(num_topk),              \
        flags, topk_divisor.magic, topk_divisor.shift, static_cast<uint32_t>(side_blocks))
        if (num_topk == 1)
            NANOEP_LAUNCH_FEW(1);
        else if (num_topk == 2)
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
        vectors, chunks, num_topk, flags)
#define NANOEP_LAUNCH_COMBINE_GROUP(GROUP)    \
    do {                                     \
        if (direct)                          \
            NANOEP_LAUNCH_COMBINE(GROUP, true);  \
        else                                 \
            NANOEP_LAUNCH_COMBINE(GROUP, false); \
    } while (0)
    // the group size is the number of rows fetched per pass: the smallest of 1, 2, 4, 8, 16 covering K
    if (num_topk <= 1)
        NANOEP_LAUNCH_COMBINE_GROUP(1);
    else if (num_topk <= 2)
        NANOEP_LAUNCH_COMBINE_GROUP(2);
    else if (num_topk <= 4)
        NANOEP_LAUNCH_COMBINE_GROUP(4);
    else if (num_topk <= 8)
        NANOEP_LAUNCH_COMBINE_GROUP(8);
    else
        NANOEP_LAUNCH_COMBINE_GROUP(16);
#undef NANOEP_LAUNCH_COMBINE_GROUP
#undef NANOEP_LAUNCH_COMBINE
    NANOEP_HIP_TRY(hipGetLastError());
    return NANOEP_OK;
}

}  // extern "C"
