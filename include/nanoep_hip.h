/*
 * nanoep_hip.h -- C ABI of the MI355X (gfx950) expert-parallel dispatch / combine kernels.
 *
 * One rank, one GPU.  Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void* so that the header needs no HIP include), enqueues work on that stream,
 * allocates nothing, throws nothing and returns a status code (NANOEP_OK == 0).
 *
 * Shapes use the reference's letters: T source tokens, H hidden, K top-k, L local experts,
 * N received rows (tokens with at least one valid choice), C padded expanded capacity.
 *
 * The handle tensors are the seven the reference's dispatch returns
 * (csrc/include/nano_ep/pipeline.hpp:13-21 in the reference):
 *   recv_metadata  int32 [N, K+2] = [src_rank(=0), src_token, K x (local expert id | expanded slot | -1)]
 *   expert_counts  int64 [L]      actual assignments per expert
 *   expert_offsets int64 [L+1]    exclusive prefix of counts rounded up to `alignment`; [L] == C
 *   dst_slots      int64 [T, 1]   receive row of each source token, -1 when it is not sent
 *   send_counts    int64 [1]      == N
 *   topk_snapshot  int64 [T, K]   copy of the routing ids
 *   recv_rank_prefix int64 [1]    == N
 */
#ifndef NANOEP_HIP_H_
#define NANOEP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NANOEP_OK 0
#define NANOEP_ERR_INVALID_ARGUMENT 1 /* shape / pointer / alignment precondition violated */
#define NANOEP_ERR_HIP 2              /* a HIP runtime call failed; see nanoep_last_hip_error() */
#define NANOEP_ERR_WORKSPACE 3        /* workspace too small */
#define NANOEP_ERR_TIMEOUT 4          /* host wait for the layout counts timed out */
#define NANOEP_ERR_ROUTING 5          /* layout kernel saw an expert id outside [-1, L) or a duplicate */
#define NANOEP_ERR_SCRATCH_LIMIT 6    /* nanoep_layout_static: (T, K, L) needs more than NANOEP_STATIC_SCRATCH_BYTES */

/* Bits of the routing status word the layout kernels publish (host_counts[3]). */
#define NANOEP_ROUTING_BAD_EXPERT 1
#define NANOEP_ROUTING_DUPLICATE 2

/* Number of int64 words in the host mailbox passed to nanoep_layout / nanoep_wait_counts. */
#define NANOEP_HOST_COUNT_WORDS 4

int nanoep_abi_version(void);
const char* nanoep_status_string(int status);
/* hipGetErrorString of the last HIP failure seen on this thread ("" when none). */
const char* nanoep_last_hip_error(void);

/* Compute-unit count of `device` (the reference's "device SM count",
 * nano_ep/backends/cuda.py:108-109). */
int nanoep_device_cu_count(int device, int* out_cus);

/* What the launch plans take from the current device: compute units, XCDs (each with its own L2;
 * workgroups are dealt to them round-robin) and the bytes of one XCD's L2.  A process without a
 * device gets the MI355X's 256 / 8 / 4 MiB.  The XCDS and L2_BYTES switches below override the
 * last two.  No counterpart in the reference (its grids are sized by num_sms alone,
 * csrc/pipeline.cu:20-24).  Any pointer may be NULL. */
int nanoep_device_topology(int* out_cus, int* out_xcds, int64_t* out_l2_bytes);

/*
 * Tuning switches.  Each is read once per process from the environment variable NANOEP_<NAME>
 * (first use of the library); afterwards only these calls change it, so no entry point touches the
 * environment on its way to a launch.  Meant for tests and sweeps: the defaults are the measured
 * best.  No counterpart in the reference.
 *   CHUNKS_PER_BLOCK, ROWS_PER_BLOCK (0: by shape)  workgroup shape of the row kernels (the slot-order
 *                     walk takes ROWS_PER_BLOCK list entries a workgroup for rows of up to 4 KiB)
 *   DISPATCH_ORDER (-1; 0: token-order walk even when the handle has a slot-order list)
 *   DISPATCH_SPAN (0: by size; 1 | 2 | 4 chunks a wavefront of the slot-order walk)
 *   DISPATCH_PACK (0: rows of at most 512 / 256 bytes go four / eight list entries a wavefront in
 *                     that walk; 1: one entry a wavefront whatever the row length)
 *   DISPATCH_PREFETCH (-1: on; 0: no window-wise source prefetch in that walk, for sources that are
 *                     known to sit in the last-level cache)
 *   COMBINE_STORES (-1: by output size; 0 | 1: nontemporal / agent-scope stores for the combine's output)
 *   COMBINE_UNITS (0: by size; 1 .. 16 tokens a wavefront of the expanded combine with five or more
 *                     rows a token and the slot table; 1 = the one-token kernel)
 *   LAYOUT_LAUNCHES (0; 2 | 3: layout plan)     WINDOW_TOKENS (0; window of the slot-order list)
 *   RECALL_ORDER, FRESH_OUTPUTS, REBUILD_ORDER (-1; 0 | 1: host-extension policies)
 *   XCDS, L2_BYTES (0: ask the device)
 * nanoep_set_tuning / nanoep_get_tuning return NANOEP_ERR_INVALID_ARGUMENT for an unknown name;
 * nanoep_reset_tuning reads every switch from the environment again.
 */
int nanoep_set_tuning(const char* name, int value);
int nanoep_get_tuning(const char* name, int* value);
void nanoep_reset_tuning(void);

/* Byte offsets of the reference's peer window regions; a pure function kept so that a caller
 * written against csrc/bindings.cpp:47-58 / csrc/layout.hpp:59-98 still finds it.
 * out = {signal_offset, count_offset, payload_offset, return_offset, num_bytes}. */
int nanoep_window_layout(int ranks, int64_t max_tokens, int hidden, int topk, int64_t num_experts,
                         int allow_multiple_reduction, int64_t out[5]);

/* Device scratch needed by nanoep_layout for (T, K, L). */
size_t nanoep_layout_workspace_bytes(int64_t num_tokens, int num_topk, int64_t num_local_experts);

/* Tokens of one block ("window") of the slot-order list for T tokens, L local experts and payload
 * rows of `hidden` bf16 elements (0: not known; the answer is 0 when L is not supported).  The list
 * is ordered window of consecutive tokens by window, and a window's rows should fit one XCD's 4 MiB
 * L2: 512 tokens up to hidden 4096 (1024 tokens up to hidden 1024), 256 up to 8192 (and when hidden
 * is not known), then 128 and 64; fewer for batches of 257..4095 tokens so that there are eight
 * windows (sixteen before a window takes 1024 tokens), and the layout workgroup's
 * own token count when the layout needs its separate scan launch (more than 1024 workgroups). */
int nanoep_layout_block_tokens(int64_t num_tokens, int64_t num_local_experts, int hidden);

/* Number of int64 words of the slot-order buffer for (T, K, L): T rounded up to 256, times K
 * entries (an upper bound of the A that carry assignments), then one word holding A.  0 when T == 0. */
int64_t nanoep_slot_order_entries(int64_t num_tokens, int num_topk, int64_t num_local_experts);

/*
 * Routing layout: histogram + device-wide exclusive scan + stable token-order slot assignment.
 * Replaces count_and_notify / finalize_receive_counts (csrc/dispatch_main.cuh:116-210, :70-114),
 * the send-slot assignment of dispatch_payload_rows (csrc/dispatch_main.cuh:278-311) and
 * build_receive_metadata_row (csrc/dispatch_epilogue.cuh:20-47); results follow
 * reference_layout (nano_ep/testing/oracle.py:70-104) with rows and slots in token order.
 *
 * Limits: T <= 2^31 - 1, K <= 32, L <= 3839 (the assignment kernel keeps four int32 per expert in
 * LDS), alignment <= 2^31; anything beyond returns NANOEP_ERR_INVALID_ARGUMENT.
 * recv_metadata must have room for T rows; the first N are written.
 * token_slots (optional, int32 [T, K]) receives slot[t,k] (or the local id when !expand), -1 when
 * masked: the same information as dst_slots + recv_metadata in one lookup.  It is not one of the
 * reference's handle tensors; nanoep_dispatch / nanoep_combine run a little faster when given it.
 * slot_order (optional, expanded only, T*K < 2^31, int64 [nanoep_slot_order_entries]) lists the A
 * valid assignments as (slot << 32) | (t * K + k), token block by token block and in ascending slot
 * (that is expert-major) order inside a block; the entries from A on are -1 and the last word of
 * the buffer holds A.  Walking it makes a dispatch write runs of consecutive destination
 * rows while a block's source rows stay cache resident.  Like token_slots it is private to this library.
 * hidden is the row width (bf16 elements) of the payload that will be dispatched with this handle,
 * 0 when not known: it only sizes the token blocks (nanoep_layout_block_tokens).
 * host_counts is pinned, device-visible host memory of NANOEP_HOST_COUNT_WORDS int64:
 * the call sets word 0 to -1, the device later stores {N, C, A (total assignments), status}
 * with word 0 last, so a host that sees word 0 >= 0 may read the rest.
 */
int nanoep_layout(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts,
                  int64_t alignment, int expand, int hidden, int32_t* recv_metadata, int64_t* expert_counts,
                  int64_t* expert_offsets, int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot,
                  int64_t* recv_rank_prefix, int32_t* token_slots, int64_t* slot_order, void* workspace,
                  size_t workspace_bytes, int64_t* host_counts, void* stream);

/* Size of the device array behind nanoep_layout_static (4 MiB on every GPU the library runs on). */
#define NANOEP_STATIC_SCRATCH_BYTES (4u << 20)

/*
 * nanoep_layout without the workspace arguments, for callers that cannot allocate device memory
 * (tight serving loops, harnesses that forbid hipMalloc, code that records its launches into a HIP
 * graph).  It has no counterpart in the reference.  A caller that captures it must know two things:
 * the first call on a device resolves the array's address through the runtime and belongs outside
 * the capture, and the -1 this call stores into host_counts[0] is a host store made when the call
 * is made, not part of the graph: before every launch of the graph the caller stores -1 there
 * itself, or nanoep_wait_counts answers with the previous launch's counts.  The kernels' workspace is a file-scope device array of
 * NANOEP_STATIC_SCRATCH_BYTES that each GPU holds until the process ends; the call allocates
 * and frees nothing (its first call on a device looks the array's address up once).  Inputs, outputs
 * and results are those of nanoep_layout.  A geometry whose workspace
 * (nanoep_layout_workspace_bytes) exceeds the array returns NANOEP_ERR_SCRATCH_LIMIT before anything
 * is enqueued: 4096 tokens x top-8 x 256 experts need 0.2 MiB, 32768 tokens 1.7 MiB.
 * All calls on one GPU share the one array: two calls whose kernels can overlap in time (different
 * streams, or different threads) race and must be serialized by the caller.
 */
int nanoep_layout_static(const int64_t* topk_idx, int64_t num_tokens, int num_topk, int64_t num_local_experts,
                         int64_t alignment, int expand, int hidden, int32_t* recv_metadata, int64_t* expert_counts,
                         int64_t* expert_offsets, int64_t* dst_slots, int64_t* send_counts, int64_t* topk_snapshot,
                         int64_t* recv_rank_prefix, int32_t* token_slots, int64_t* slot_order, int64_t* host_counts,
                         void* stream);

/* Tokens of one window of the list nanoep_rebuild_order writes for (T, K, hidden). */
int nanoep_rebuild_window_tokens(int64_t num_tokens, int num_topk, int hidden);

/* Device scratch needed by nanoep_rebuild_order for (T, K). */
size_t nanoep_rebuild_workspace_bytes(int64_t num_tokens, int num_topk);

/*
 * The two private handle tensors of an expanded handle, rebuilt from its public ones alone: for a
 * handle that comes back with only the seven tensors the reference's operator boundary carries
 * (csrc/pipeline.cu:357-358, nano_ep/backends/cuda.py:296-304).  The handle is followed as it is
 * written, whatever order its rows and slots are in (the reference's own helper builds handles in
 * another order, nano_ep/testing/native_combine.py:62-74):
 *   token_slots[t][k] = recv_metadata[dst_slots[t]][2 + k], -1 when the token was not sent or the
 *                       value lies outside [0, expanded_capacity)
 *   slot_order        = window of consecutive tokens by window, the valid (slot << 32) | (t * K + k)
 *                       in ascending slot order, -1 from entry A on, A in the buffer's last word
 * (a window is nanoep_layout_block_tokens' for `hidden`, halved until its T * K entries number at
 * most 4096: any window size is a valid list, the size only decides the walk's locality).
 * token_slots is int32 [T, K], slot_order int64 [nanoep_slot_order_entries]; workspace needs
 * nanoep_rebuild_workspace_bytes.  host_count, when not NULL, is one pinned int64 the host can read:
 * the call stores -1 there and the device later stores host_tag | A (host_tag: a non-negative number
 * with its low 32 bits clear, so that a reader can tell this call's answer from an older one's).
 * Two launches on `stream`; T * K < 2^31, T > 0.
 */
int nanoep_rebuild_order(const int32_t* recv_metadata, const int64_t* dst_slots, int64_t recv_count, int64_t expanded_capacity,
                         int64_t num_tokens, int num_topk, int64_t num_local_experts, int hidden, int32_t* token_slots,
                         int64_t* slot_order, void* workspace, size_t workspace_bytes, int64_t* host_count, int64_t host_tag,
                         void* stream);

/* Spin on the mailbox until the layout enqueued on `stream` has published its counts
 * (the reference's wait_dispatch_counts, csrc/peer.cu:198-227).  out = {N, C, A, status}. */
int nanoep_wait_counts(int64_t* host_counts, void* stream, double timeout_seconds,
                       int64_t out[NANOEP_HOST_COUNT_WORDS]);

/*
 * Dispatch permute / expand.  Replaces dispatch_payload_rows + dispatch_epilogue_kernel +
 * do_zero_padding (csrc/dispatch_main.cuh:215-354, csrc/dispatch_epilogue.cuh:123-250, :50-117);
 * results follow reference_dispatch (nano_ep/testing/oracle.py:107-147).
 *   compact : recv_x[row] = x[t]; recv_topk_idx[row,:] = local ids; recv_weights[row,:] = weights[t,:]
 *   expanded: recv_x[slot] = x[t]; recv_weights[slot] = weights[t,k]; with zero_padding the rows
 *             [offsets[e]+counts[e], offsets[e+1]) and their weights are zero-filled.
 * Work is walked in source-token order: dst_slots[t] names the receive row whose metadata holds
 * the token's slots (token_slots, when not NULL and expanded, replaces that two-step lookup).
 * When slot_order is given for an expanded dispatch, the work is walked in that order instead and
 * neither of the other lookups is read for the payload.  slot_order_entries is A when the caller
 * knows it (the list may then be just its first A entries); a caller that enqueues the dispatch
 * before it has read the counts passes a negative number with the full buffer, and the kernel takes
 * A from the buffer's last word: -1 sizes the launch for the most entries the list can hold (T * K),
 * -g (g > 1) for about g entries, which is cheaper when many choices are masked and correct whatever
 * A turns out to be (workgroups then take several turns).
 * The slot-order walk reads every window's source rows front to back just ahead of the window's
 * copies (unless the DISPATCH_PREFETCH switch is 0): the same bytes from HBM, as one sequential burst
 * per window instead of one row at a time among the stores.  It serves lists of fewer than 2^29
 * entries and rows of up to 64 KiB; beyond either the work is walked in source-token order.
 * x / recv_x are bf16, 16-byte aligned, H % 8 == 0.  weights / recv_weights / recv_topk_idx may be
 * NULL (recv_topk_idx must be NULL when expanded).  num_cus is the reference's SM budget
 * (0 = whole device): it is range-checked against the device's compute-unit count and otherwise
 * ignored here, because these kernels are sized by the work, not by a cooperative grid; a caller
 * that wants the kernels confined to fewer compute units passes a stream created with a CU mask
 * (hipExtStreamCreateWithCUMask), as the host extension does.
 */
int nanoep_dispatch(const void* x, const float* weights, const int32_t* recv_metadata, const int64_t* dst_slots,
                    const int32_t* token_slots, const int64_t* slot_order, int64_t slot_order_entries,
                    const int64_t* expert_counts, const int64_t* expert_offsets, int64_t recv_count, int64_t expanded_capacity, int64_t num_tokens, int hidden, int num_topk,
                    int64_t num_local_experts, int64_t alignment, int expand, int zero_padding, void* recv_x,
                    int64_t* recv_topk_idx, float* recv_weights, int num_cus, void* stream);

/*
 * Combine gather-reduce.  Replaces combine_return_rows + combine_epilogue_kernel
 * (csrc/combine_main.cuh:38-246, csrc/combine_epilogue.cuh:58-202); results follow
 * reference_combine (nano_ep/testing/oracle.py:150-186) and reference_combined
 * (nano_ep/testing/native_combine.py:168-195) for one rank:
 *   out_x[t] = bf16_rne( sum over valid k ascending of f32(y[slot[t,k]]) (+ f32(bias[t])) )
 * (compact: the single row y[row(t)]); tokens that were not sent get 0 (+bias).
 * multiple_reduction != 0 with expand rounds the sum of two or more rows to bf16 once before
 * the final fp32 pass, as the reference's allow_multiple_reduction mode does.
 * out_weights[t,k] = valid ? (expand ? weights[slot] : weights[row,k]) : 0.
 * y_rows is the row count of y (C when expanded, N when compact).
 * num_cus (0 = whole device) is range-checked like the dispatch's; the expanded combine with five or
 * more rows a token and the slot table also sizes its launch by it (its wavefronts hold the sums of
 * several tokens, as many as it takes for the launch to fit the wavefronts that many compute units
 * hold at once), so a caller that confines the call with a CU-masked stream passes the mask's count.
 */
int nanoep_combine(const void* y, const float* weights, const void* bias, const int32_t* recv_metadata,
                   const int64_t* dst_slots, const int32_t* token_slots, int64_t recv_count, int64_t y_rows,
                   int64_t num_tokens, int hidden, int num_topk, int expand, int multiple_reduction, void* out_x,
                   float* out_weights, int num_cus, void* stream);

/*
 * Plain streams in the shape of the row kernels (one wavefront per KiB of a destination row of
 * `hidden` bf16 elements, workgroups of waves_per_block consecutive KiB, 0: a workgroup per row;
 * addresses a closed form of the workgroup index, no lookups): the measured ceiling for a permute of
 * the same bytes.  No counterpart in the reference.
 *   kind 0: read dst_rows rows of src (dst is only written if a lane reads one impossible bit pattern)
 *   kind 1: fill dst_rows rows of dst
 *   kind 2: fan-out.  Source rows go in windows of `window` rows, each written `fan` times in `fan`
 *           passes over the window: dst row w * window * fan + p * window + i = src row w * window + i
 *           (src has dst_rows / fan rows; window 1: fan neighbouring rows share their source row)
 *   kind 3: fan-in.  dst row w * window + i = integer sum of the src rows
 *           w * window * fan + p * window + i, p < fan (src has dst_rows * fan rows)
 * hidden <= 8192; fan 1, 2, 4, 7 or 8; dst_rows a multiple of window * fan (kind 2) or window (kind 3).
 */
int nanoep_stream_probe(int kind, const void* src, void* dst, int64_t dst_rows, int hidden, int fan, int64_t window,
                        int waves_per_block, void* stream);

/* Plain 16-byte-vector device copy of `bytes` (multiple of 16); the known-size kernel used to
 * scale the profiler's HBM byte counters.  No counterpart in the reference. */
int nanoep_copy_bytes(const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* NANOEP_HIP_H_ */
