// MI355X (gfx950, wave64) kernels for one rank's expert-parallel dispatch / combine, and the
// C ABI declared in include/nanoep_hip.h: nanoep_layout.hip, nanoep_dispatch.hip,
// nanoep_combine.hip, nanoep_abi.hip.  This header holds what they share.
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
//   dispatch_walk_kernel : expanded layouts with the layout's slot-order list: one wavefront per
//                          (list entry, row chunk), window of tokens by window and expert-major
//                          inside a window, so a window's source rows stay in one XCD's L2 and every
//                          expert receives runs of consecutive rows; one 128-bit load and one
//                          nontemporal 128-bit store per lane, as few scalar instructions ahead of
//                          the load as the work allows.  A few workgroups ahead of every window read
//                          its source rows front to back (prefetch).
//   dispatch_rows_kernel : the same work item walked in source-token order (small batches, handles
//                          without the list); extra work items zero-fill the alignment gaps.
//   dispatch_compact_kernel / combine_compact_kernel : compact layouts are row copies with holes;
//                          plain launch order, single-wavefront workgroups, nothing but the copy.
//   combine_rows_kernel  : one wavefront per (source token, row chunk): gathers the token's rows in
//                          ascending k, fp32 accumulate, one round-to-nearest-even bf16 store.
//   combine_few_rows_kernel : the same for K <= 4 with the slot table, without the bookkeeping.
//   combine_held_kernel  : the same for K > 4 with the slot table: a wavefront sums its chunk of 2
//                          to 16 consecutive tokens' rows and writes them all at its end, so that a
//                          launch whose wavefronts are all resident reads first and writes last.
//   rebuild_table_kernel + rebuild_order_kernel : the slot table and the slot-order list of a handle
//                          rebuilt from its recv_metadata and dst_slots alone (an LDS bitonic sort
//                          of every window's (slot, source) pairs).
//   stream_probe_kernel  : plain streams in the shape of the row kernels (measured ceilings).
//
// Every byte moved is HBM-bound integer/byte work; there is no contraction, hence no MFMA.
#ifndef NANOEP_DEVICE_H_
#define NANOEP_DEVICE_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "nanoep_hip.h"

namespace nanoep {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWave * kWavesPerBlock;
constexpr int kScanThreads = 1024;
constexpr int kMaxTopk = 32;
constexpr size_t kLayoutLdsBudget = 60 * 1024;

// Last HIP failure seen on this thread (nanoep_last_hip_error reports it); defined in nanoep_abi.hip.
extern thread_local hipError_t g_last_hip_error;

#define NANOEP_HIP_TRY(expr)              \
    do {                                  \
        const hipError_t status_ = (expr); \
        if (status_ != hipSuccess) {      \
            ::nanoep::g_last_hip_error = status_;   \
            return NANOEP_ERR_HIP;        \
        }                                 \
    } while (0)

inline size_t align_up(size_t value, size_t alignment) { return (value + alignment - 1) / alignment * alignment; }

// Tuning switches of the library.  Each is NANOEP_<NAME> in the environment, which is read exactly
// once per process, on the first use of the library; nanoep_set_tuning changes one afterwards (tests
// and sweeps do that between calls).  The record is a handful of relaxed atomics: entry points take
// one snapshot of it (current_tuning) and the code below them only looks at the snapshot.
struct Tuning {
    int chunks_per_block = 0;       // CHUNKS_PER_BLOCK: wavefronts along a row in a workgroup, 0 = by shape
    int rows_per_block = 0;         // ROWS_PER_BLOCK: rows a workgroup, 0 = by shape
    int dispatch_order = -1;        // DISPATCH_ORDER: 0 forces the token-order walk
    int dispatch_span = 0;          // DISPATCH_SPAN: 1 | 2 | 4 chunks a wavefront of the slot-order walk, 0 = by size
    int dispatch_prefetch = -1;     // DISPATCH_PREFETCH: 0 = no window-wise source prefetch in the slot-order walk
    int combine_units = 0;          // COMBINE_UNITS: tokens a wavefront of the gather for five or more rows a token: 1 .. 16, 0 = by size
    int dispatch_pack = 0;          // DISPATCH_PACK: 1 = one list entry a wavefront of the slot-order walk whatever the row length
    int combine_stores = -1;        // COMBINE_STORES: 0 | 1 nontemporal / agent-scope stores for the combine's output, -1 = by size
    int layout_launches = 0;        // LAYOUT_LAUNCHES: 2 | 3 forces the layout plan
    int window_tokens = 0;          // WINDOW_TOKENS: forces the window of the slot-order list
    int recall_order = -1;          // RECALL_ORDER: 0 = seven-tensor handles never get private tensors back (host extension)
    int fresh_outputs = -1;         // FRESH_OUTPUTS: 0 | 1 where a fresh dispatch's outputs are allocated (host extension)
    int rebuild_order = -1;         // REBUILD_ORDER: 0 | 1 never / always rebuild the private tensors of a seven-tensor handle
    int xcds = 0;                   // XCDS: number of XCDs the block remap assumes, 0 = ask the device
    int l2_bytes = 0;               // L2_BYTES: size of one XCD's L2 the windows are sized for, 0 = ask the device
};

Tuning current_tuning();  // defined in nanoep_abi.hip

// What the launch plans need to know of the device: compute units, XCDs (each with an L2 of its
// own; workgroups are handed to them round-robin by linear id) and the size of one such L2.
// Asked of the runtime once per device; a process without a device gets the MI355X's numbers.
struct Topology {
    int cus = 256;
    int xcds = 8;
    int64_t l2_bytes = int64_t{4} << 20;
    // wavefronts of combine_held_kernel<2 | 4 | 8 | 16> that a compute unit holds at once
    int held_wavefronts[4] = {32, 32, 24, 16};
};

// Fills Topology::held_wavefronts from the register counts of the built kernels (nanoep_combine.hip).
void held_combine_residency(int out[4]);

Topology current_topology(const Tuning& tuning);  // defined in nanoep_abi.hip

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

// Store for rows that are written once among many reads (the combine's output): agent scope, no
// nontemporal hint.  Against the nontemporal store it measured 2 to 7 % on the combine kernels
// (4096 x 7168 top-8: 79.9 -> 78.0 us, 4096 x 4096 top-2: 18.4 -> 17.2 us); under the dispatch's
// fan-out of writes it is 60 % slower than the nontemporal one.
__device__ __forceinline__ void store_vec_agent(u32x4* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}

// Load through the scalar data path: the address must be wave-uniform and the memory read-only for
// the duration of the kernel (true of all handle tensors here).  Keeps lookups out of the vector
// memory pipeline and their results in SGPRs.
template <class T>
__device__ __forceinline__ T uniform_load(const T* p) {
    return *(const __attribute__((address_space(4))) T*)(p);
}

// Element `index` of such an array, addressed with a 32-bit byte offset (index * sizeof(T) < 2^32):
// the offset then rides in the load instruction instead of a 64-bit address computation.
template <class T>
__device__ __forceinline__ T uniform_load_at(const T* base, uint32_t index) {
    typedef const __attribute__((address_space(4))) char* ConstantBytes;
    typedef const __attribute__((address_space(4))) T* ConstantElement;
    return *(ConstantElement)((ConstantBytes)(base) + index * static_cast<uint32_t>(sizeof(T)));
}

// A uniform 64-bit load in two halves: begin issues it, end waits for it.  Between the two the value
// must not be touched; what the wavefront computes meanwhile hides the load's latency (the compiler
// on its own moves such a load down to its first use).
// `anchor` is any scalar the following arithmetic starts from: tied to the statement, it keeps that
// arithmetic behind the load's issue.
__device__ __forceinline__ int64_t uniform_load_begin(const int64_t* p, uint32_t& anchor) {
    int64_t value;
    asm volatile("s_load_dwordx2 %0, %2, 0x0" : "=s"(value), "+s"(anchor) : "s"(p));
    return value;
}
__device__ __forceinline__ int64_t uniform_load_end(int64_t value) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(value));
    return value;
}

// n / d for n < 2^31 as one 64-bit multiply and shift: magic = ceil(2^shift / d), shift = 31 + ceil(log2 d).
struct FastDivisor {
    uint32_t magic;
    uint32_t shift;
};

inline FastDivisor make_fast_divisor(uint32_t divisor) {
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

// Workgroups are handed to the XCDs round-robin by their linear id and every XCD has its own L2, so
// kernels whose neighbouring work items share data remap the linear id: workgroup b runs on XCD
// b % count and is the (b / count)-th workgroup there.  count comes from the device (8 on an
// unpartitioned MI355X), so the division is a multiply-shift by a host-made magic number.
struct XcdMap {
    uint32_t count;
    uint32_t magic;
    uint32_t shift;
};

inline XcdMap make_xcd_map(int xcds) {
    const uint32_t count = xcds > 0 ? static_cast<uint32_t>(xcds) : 1u;
    const FastDivisor divisor = make_fast_divisor(count);
    return {count, divisor.magic, divisor.shift};
}

// Kernel arguments are fetched with scalar loads where they are first used, which strings several
// dependent round trips along a short wavefront's life.  Naming them in an empty asm statement at
// the top of the kernel makes the compiler fetch them all in one batch.
#define NANOEP_FETCH_ARGS_2(a, b) asm volatile("" ::"s"(a), "s"(b))
#define NANOEP_FETCH_ARGS_4(a, b, c, d) asm volatile("" ::"s"(a), "s"(b), "s"(c), "s"(d))

// Last-level (memory-side) cache of the MI355X: 256 MiB.
constexpr int64_t kLastLevelCacheBytes = int64_t{256} << 20;

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
    kRowCopyWalk,     // compact layouts (plain row copies): single-wavefront workgroups
};

inline RowBlocking pick_row_blocking(int chunks, WalkShape shape, const Tuning& tuning) {
    RowBlocking blocking{};
    int per_block = tuning.chunks_per_block;
    if (per_block < 1 || per_block > kMaxWavesPerBlock)
        per_block = shape == kRowCopyWalk ? 1 : kDefaultChunksPerBlock;
    if (per_block > chunks)
        per_block = chunks;
    blocking.chunks_per_block = static_cast<unsigned>(per_block);
    blocking.parts = static_cast<unsigned>((chunks + per_block - 1) / per_block);
    int rows = 1;
    if (blocking.parts == 1) {
        rows = tuning.rows_per_block;
        if (rows < 1 || rows * per_block > kMaxWavesPerBlock)
            rows = per_block >= 4 ? 1 : 4 / per_block;
    }
    blocking.rows_per_block = static_cast<unsigned>(rows);
    return blocking;
}

// List entries a workgroup of the slot-order walk takes when a row has up to four pieces (longer
// rows take a workgroup each, one wavefront a piece).
inline int default_walk_rows(int pieces) {
    return pieces == 3 ? 1 : pieces == 1 ? 4 : 2;
}

inline int validate_cu_budget(int num_cus, const Topology& topology) {
    return (num_cus < 0 || num_cus > topology.cus) ? NANOEP_ERR_INVALID_ARGUMENT : NANOEP_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace nanoep

#endif  // NANOEP_DEVICE_H_
