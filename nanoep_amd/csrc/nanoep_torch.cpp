// PyTorch-ROCm host extension for one rank's dispatch / combine.
//
// This file owns what the reference's host pipeline owns (csrc/pipeline.cu:340-489,
// csrc/dispatch_epilogue.cpp:18-75, csrc/combine_epilogue.cpp:27-64 in the reference): argument
// validation, output allocation, stream ordering between the caller's stream and the buffer's
// communication stream, and the completion event.  All device work goes through the C ABI of
// include/nanoep_hip.h.  The module exports the reference's operator surface
// (csrc/bindings.cpp:11-86) with the same positional order, so a caller written against the
// reference's backend module binds to this one unchanged.

#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/Event.h>
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <array>
#include <atomic>
#include <cstdlib>
#include <deque>
#include <limits>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "nanoep_hip.h"

namespace py = pybind11;

namespace nanoep {

using Stream = c10::hip::HIPStreamMasqueradingAsCUDA;
using StreamGuard = c10::hip::HIPStreamGuardMasqueradingAsCUDA;
using OptionalStreamGuard = c10::hip::OptionalHIPStreamGuardMasqueradingAsCUDA;
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

namespace {

constexpr int64_t kHiddenAlignment = 256;  // the reference's H % 256 == 0 contract
constexpr double kCountTimeoutSeconds = 60.0;
// Fresh expanded dispatches whose private handle tensors the runtime keeps for callers that hand
// back only the reference's seven.
constexpr size_t kRememberedHandles = 4;
// Seven-tensor handles whose private tensors were rebuilt from the handle itself and are kept for
// its later replays.
constexpr size_t kRebuiltHandles = 64;
// Rebuilding pays from this many payload bytes written per replay on (below, the token-order walk's
// loss is smaller than what the two extra launches cost a handle that is replayed once or twice).
constexpr int64_t kRebuildPayloadBytes = int64_t{48} << 20;

// One of the library's tuning switches (no environment access: the library read it once).
int tuning_switch(const char* name) {
    int value = -1;
    return nanoep_get_tuning(name, &value) == NANOEP_OK ? value : -1;
}

void check_status(int status, const char* what) {
    if (status == NANOEP_OK)
        return;
    TORCH_CHECK(false, "nanoep ", what, " failed: ", nanoep_status_string(status), " ", nanoep_last_hip_error());
}

void check_hip(hipError_t status, const char* what) {
    TORCH_CHECK(status == hipSuccess, "HIP call ", what, " failed: ", hipGetErrorString(status));
}

Stream external_stream(int64_t handle, c10::DeviceIndex device) {
    return c10::hip::getStreamFromExternalMasqueradingAsCUDA(reinterpret_cast<hipStream_t>(handle), device);
}

void wait_on(const Stream& waiter, const Stream& producer) {
    c10::Event ready(c10::DeviceType::CUDA);
    ready.record(producer.unwrap());
    waiter.unwrap().wait(ready);
}

// Compute-unit budget: 0 or the device size mean the whole device (the reference's
// resolve_main_sms, csrc/pipeline.cu:20-24).
int resolve_cu_budget(int num_sms, c10::DeviceIndex device) {
    const int device_cus = at::cuda::getDeviceProperties(device)->multiProcessorCount;
    TORCH_CHECK(num_sms >= 0 && num_sms <= device_cus, "num_sms must be between 0 and the device CU count (", device_cus, ")");
    return num_sms == device_cus ? 0 : num_sms;
}

}  // namespace

// Holds what one rank needs at world_size == 1: the device, the pinned host mailbox the layout
// kernels publish N / C into, and (only if somebody asks for it) a window-sized byte tensor.
// It keeps the reference's PeerRuntime method set (csrc/bindings.cpp:59-83) so setup code written
// for the reference runs; there are no peers, so handles are opaque tags and barriers are no-ops.
//
// dispatch and combine run without the interpreter lock, so everything here that several Python
// threads can reach at once is guarded: the mailbox by `counts_mutex_` (held by a fresh dispatch
// from the enqueue of its layout until it has read the counts), the remembered handle tensors by
// `private_mutex_`, the state flags by being atomic.
class PeerRuntime {
   public:
    PeerRuntime(int rank, int world_size, int64_t num_bytes) : num_bytes_(num_bytes) {
        TORCH_CHECK(world_size == 1 && rank == 0,
                    "this build runs one rank on one GPU (world_size == 1); got rank ", rank, " of ", world_size);
        TORCH_CHECK(num_bytes >= 0, "window size must be non-negative");
        check_hip(hipGetDevice(&device_), "hipGetDevice");
        void* mailbox = nullptr;
        check_hip(hipHostMalloc(&mailbox, NANOEP_HOST_COUNT_WORDS * sizeof(int64_t), hipHostMallocMapped | hipHostMallocCoherent),
                  "hipHostMalloc");
        host_counts_ = static_cast<int64_t*>(mailbox);
        for (int i = 0; i < NANOEP_HOST_COUNT_WORDS; ++i)
            host_counts_[i] = -1;
        void* words = nullptr;
        check_hip(hipHostMalloc(&words, kRebuiltHandles * sizeof(int64_t), hipHostMallocMapped | hipHostMallocCoherent), "hipHostMalloc");
        rebuilt_counts_ = static_cast<int64_t*>(words);
        for (size_t i = 0; i < kRebuiltHandles; ++i)
            rebuilt_counts_[i] = -1;
    }

    ~PeerRuntime() {
        if (host_counts_ != nullptr)
            (void)hipHostFree(host_counts_);
        if (rebuilt_counts_ != nullptr)
            (void)hipHostFree(rebuilt_counts_);
    }

    PeerRuntime(const PeerRuntime&) = delete;
    PeerRuntime& operator=(const PeerRuntime&) = delete;

    int rank() const { return 0; }
    int world_size() const { return 1; }
    int device() const { return device_; }

    // Every operation starts here (the reference's reserve_barrier_epochs, csrc/peer.cu:171-175):
    // a closed runtime, and one whose last fresh dispatch never got its counts, serve nothing.
    void require_usable() const {
        TORCH_CHECK(!closed_.load(), "PeerRuntime is closed");
        TORCH_CHECK(!counts_failed_.load(), "A fresh dispatch on this runtime failed while waiting for its counts; the runtime is unusable");
    }

    // One fresh dispatch's use of the mailbox, from before its layout is enqueued until the host has
    // read N and C (the reference's prepare_dispatch_counts / wait_dispatch_counts /
    // fail_dispatch_counts, csrc/peer.cu:187-232).  Fresh dispatches of other threads wait their
    // turn at the constructor.  A turn that ends without `wait` having delivered the counts (a
    // timeout, a HIP error, an exception in between) leaves the runtime failed for good: a word the
    // device stores late must never answer a later call.
    class CountsTurn {
       public:
        explicit CountsTurn(PeerRuntime& runtime) : runtime_(runtime), lock_(runtime.counts_mutex_) {
            runtime_.require_usable();
            TORCH_CHECK(!runtime_.counts_pending_.load(), "A fresh dispatch is waiting for counts or has failed");
            runtime_.counts_pending_.store(true);
        }
        CountsTurn(const CountsTurn&) = delete;
        CountsTurn& operator=(const CountsTurn&) = delete;
        ~CountsTurn() {
            if (!settled_)
                runtime_.counts_failed_.store(true);
            runtime_.counts_pending_.store(false);
        }

        int64_t* mailbox() const { return runtime_.host_counts_; }

        // Nothing was enqueued that could still write the mailbox: the turn ends without a verdict.
        void abandon() { settled_ = true; }

        // Spins until the layout enqueued on `stream` has published {N, C, A, status}.  Returns
        // NANOEP_OK or NANOEP_ERR_ROUTING (the words are complete either way); anything else throws
        // and latches the failure.
        int wait(hipStream_t stream, double timeout_seconds, int64_t (&counts)[NANOEP_HOST_COUNT_WORDS]) {
            const int status = nanoep_wait_counts(mailbox(), stream, timeout_seconds, counts);
            if (status == NANOEP_OK || status == NANOEP_ERR_ROUTING) {
                settled_ = true;
                return status;
            }
            check_status(status, "wait_counts");
            return status;
        }

       private:
        PeerRuntime& runtime_;
        std::unique_lock<std::mutex> lock_;
        bool settled_ = false;
    };

    bool counts_failed() const { return counts_failed_.load(); }

    // What a fresh dispatch whose counts never arrive leaves behind, without making a GPU misbehave:
    // a turn at the mailbox that ends with no verdict.  For tests of the failure latch.
    void lose_counts_for_test() { CountsTurn lost(*this); }

    // Whether fresh dispatches should allocate their outputs after the counts are known: set when a
    // call that allocated at the upper bound turned out to hold over 1.25 times what it used (many
    // masked choices), cleared when an exact call shows that the bound would have been close enough.
    bool prefers_exact_outputs() const { return prefers_exact_outputs_.load(); }
    void note_output_fill(bool bound_was_close) { prefers_exact_outputs_.store(!bound_was_close); }

    // Rows the latest fresh dispatch of a geometry ended up using.  Where the upper bound of the output
    // shapes is not close (large alignment gaps), a fresh dispatch of the same geometry allocates its
    // outputs for that many rows plus an eighth, launches its permute behind the layout and keeps the
    // result if the rows in use fit and fill at least four fifths of it; otherwise it permutes again
    // into exact outputs, as a first call of a geometry does.  Read and written with the mailbox held.
    struct OutputForecast {
        int64_t tokens = -1, topk = 0, experts = 0, alignment = 0, hidden = 0;
        bool expand = false;
        int64_t used_rows = 0;
    };
    int64_t forecast_rows(const OutputForecast& key) const {
        const OutputForecast& seen = forecast_;
        if (seen.tokens != key.tokens || seen.topk != key.topk || seen.experts != key.experts || seen.alignment != key.alignment ||
            seen.hidden != key.hidden || seen.expand != key.expand || seen.used_rows <= 0)
            return 0;
        return seen.used_rows + (seen.used_rows + 7) / 8;
    }
    void note_used_rows(OutputForecast key, int64_t used_rows) {
        key.used_rows = used_rows;
        forecast_ = key;
    }

    // Share of the routing choices that were valid in the latest fresh expanded dispatch, in 1/65536
    // (65536 before the first one).  A permute that is enqueued before the host knows the count sizes
    // its launch for this share of T * K plus half a percent instead of for all of it (a workgroup
    // that finds nothing to do costs about as much as one that takes a second turn, so the launch
    // aims at the count itself); any count is handled.
    int64_t valid_share_65536() const { return valid_share_65536_.load(); }
    void note_valid_share(int64_t assignments, int64_t choices) {
        if (choices > 0)
            valid_share_65536_.store((assignments * 65536 + choices - 1) / choices);
    }

    // The private handle tensors (slot table, slot-order list) of the latest few fresh expanded
    // dispatches.  A caller that keeps only the reference's seven handle tensors gets them back on
    // a replay of one of those handles: an entry is recognised by the identity of the handle's
    // routing snapshot (the tensor object, its data pointer and version) and of its recv_metadata
    // storage.  The two tensors are views of the allocation that backs the seven public ones.
    // Handles this runtime did not make, or made too long ago, are never matched: their replays
    // follow the handle's own recv_metadata and dst_slots in token order.
    void remember_private(const std::vector<torch::Tensor>& metadata, int64_t alignment) {
        if (metadata.size() < 9 || !metadata[7].defined() || !metadata[8].defined())
            return;
        RememberedHandle entry;
        entry.snapshot.emplace(metadata[5].getIntrusivePtr());
        entry.version = tensor_version(metadata[5]);
        entry.snapshot_data = metadata[5].data_ptr();
        entry.metadata_data = metadata[0].data_ptr();
        entry.rows = metadata[0].size(0);
        entry.alignment = alignment;
        entry.table = metadata[7];
        entry.order = metadata[8];
        std::vector<RememberedHandle> retired;  // released after the lock: a tensor's release may want the interpreter lock
        {
            std::lock_guard<std::mutex> lock(private_mutex_);
            // handles whose routing snapshot is gone can never come back
            for (auto it = remembered_.begin(); it != remembered_.end();) {
                if (it->snapshot->expired()) {
                    retired.push_back(std::move(*it));
                    it = remembered_.erase(it);
                } else {
                    ++it;
                }
            }
            remembered_.push_front(std::move(entry));
            while (remembered_.size() > kRememberedHandles) {
                retired.push_back(std::move(remembered_.back()));
                remembered_.pop_back();
            }
        }
    }

    // Appends the remembered private tensors to a seven-tensor handle when it is a remembered one
    // (alignment < 0: the caller does not know the handle's alignment, the identity decides).
    bool recall_private(std::vector<torch::Tensor>& metadata, int64_t alignment) const {
        std::lock_guard<std::mutex> lock(private_mutex_);
        if (closed_.load() || metadata.size() != 7)
            return false;
        for (const auto& entry : remembered_) {
            const auto alive = entry.snapshot->lock();
            if (!alive || alive.get() != metadata[5].unsafeGetTensorImpl() || metadata[5].data_ptr() != entry.snapshot_data ||
                tensor_version(metadata[5]) != entry.version || metadata[0].data_ptr() != entry.metadata_data ||
                metadata[0].size(0) != entry.rows || (alignment >= 0 && alignment != entry.alignment))
                continue;
            metadata.push_back(entry.table);
            metadata.push_back(entry.order);
            ++private_recalls_;
            return true;
        }
        return false;
    }

    // number of seven-tensor handles that got their private tensors back (for tests)
    int64_t private_recalls() const {
        std::lock_guard<std::mutex> lock(private_mutex_);
        return private_recalls_;
    }

    void forget_private() {
        std::deque<RememberedHandle> retired;
        std::array<std::shared_ptr<RebuiltHandle>, kRebuiltHandles> retired_rebuilt;
        std::lock_guard<std::mutex> lock(private_mutex_);
        retired.swap(remembered_);
        retired_rebuilt.swap(rebuilt_);
    }

    // The private tensors of a seven-tensor handle, rebuilt from the handle's own dst_slots and
    // recv_metadata (nanoep_rebuild_order) and kept for its later replays.  An entry is recognised
    // like a remembered one, and in addition by the identity and version of the two tensors it was
    // built from: a handle edited through torch is rebuilt.  `count` is where the device publishes the
    // number of list entries (tagged, so that a late store of an entry that used this word before is
    // never taken for this one's): until it is there, replays read the count on the device.
    struct RebuiltHandle {
        c10::weak_intrusive_ptr<c10::TensorImpl> snapshot;
        uint32_t snapshot_version = 0, metadata_version = 0, slots_version = 0;
        const void* snapshot_data = nullptr;
        const void* metadata_data = nullptr;
        const void* slots_data = nullptr;
        int64_t rows = 0, capacity = 0;
        torch::Tensor table, order;  // views of one allocation
        c10::Event ready{c10::DeviceType::CUDA};
        hipStream_t made_on = nullptr;
        int64_t* count = nullptr;  // pinned host word
        int64_t tag = 0;

        explicit RebuiltHandle(const torch::Tensor& snapshot_tensor) : snapshot(snapshot_tensor.getIntrusivePtr()) {}

        // the number of list entries once the device has published it, else -1
        int64_t published_entries() const {
            const int64_t word = __atomic_load_n(count, __ATOMIC_ACQUIRE);
            return word >= 0 && (word & ~int64_t{0xffffffff}) == tag ? (word & int64_t{0xffffffff}) : -1;
        }
    };

    std::shared_ptr<RebuiltHandle> find_rebuilt(const std::vector<torch::Tensor>& metadata, int64_t capacity) const {
        std::lock_guard<std::mutex> lock(private_mutex_);
        if (closed_.load() || metadata.size() != 7)
            return nullptr;
        for (const auto& entry : rebuilt_) {
            if (!entry)
                continue;
            const auto alive = entry->snapshot.lock();
            if (alive && alive.get() == metadata[5].unsafeGetTensorImpl() && metadata[5].data_ptr() == entry->snapshot_data &&
                tensor_version(metadata[5]) == entry->snapshot_version && metadata[0].data_ptr() == entry->metadata_data &&
                tensor_version(metadata[0]) == entry->metadata_version && metadata[3].data_ptr() == entry->slots_data &&
                tensor_version(metadata[3]) == entry->slots_version && metadata[0].size(0) == entry->rows && capacity == entry->capacity)
                return entry;
        }
        return nullptr;
    }

    // A new entry for this handle (tensors not yet set, not yet findable), with a count word and tag of
    // its own.  It takes the place of an entry whose handle is gone, else of the oldest one;
    // publish_rebuilt makes it findable once its tensors are there.
    std::shared_ptr<RebuiltHandle> new_rebuilt(const std::vector<torch::Tensor>& metadata, int64_t capacity) {
        auto entry = std::make_shared<RebuiltHandle>(metadata[5]);
        entry->snapshot_version = tensor_version(metadata[5]);
        entry->metadata_version = tensor_version(metadata[0]);
        entry->slots_version = tensor_version(metadata[3]);
        entry->snapshot_data = metadata[5].data_ptr();
        entry->metadata_data = metadata[0].data_ptr();
        entry->slots_data = metadata[3].data_ptr();
        entry->rows = metadata[0].size(0);
        entry->capacity = capacity;
        std::shared_ptr<RebuiltHandle> retired;  // released after the lock
        std::lock_guard<std::mutex> lock(private_mutex_);
        size_t at = kRebuiltHandles;
        for (size_t i = 0; i < kRebuiltHandles && at == kRebuiltHandles; ++i)
            if (!rebuilt_[i] || rebuilt_[i]->snapshot.expired())
                at = i;
        if (at == kRebuiltHandles)
            at = next_rebuilt_++ % kRebuiltHandles;
        entry->count = rebuilt_counts_ + at;
        entry->tag = (++rebuilt_generation_ & 0x3fffffff) << 32;
        retired = std::move(rebuilt_[at]);
        ++rebuilds_;
        return entry;
    }

    void publish_rebuilt(const std::shared_ptr<RebuiltHandle>& entry) {
        std::shared_ptr<RebuiltHandle> retired;  // released after the lock
        std::lock_guard<std::mutex> lock(private_mutex_);
        if (closed_.load())
            return;
        retired = std::move(rebuilt_[entry->count - rebuilt_counts_]);
        rebuilt_[entry->count - rebuilt_counts_] = entry;
    }

    // number of seven-tensor handles whose private tensors were rebuilt (for tests)
    int64_t rebuilds() const {
        std::lock_guard<std::mutex> lock(private_mutex_);
        return rebuilds_;
    }

    // Scratch of the layout kernels, kept between fresh dispatches (they take turns at the mailbox and
    // a turn ends when the layout has published its counts, but its last workgroups may still be reading
    // the scratch: the buffer is only handed out again to a call on the stream it was last used on,
    // where the launches are ordered; a call on another stream gets a buffer of its own, which is then
    // the one that is kept).  Called with the mailbox held.
    torch::Tensor layout_workspace(size_t bytes, hipStream_t stream, const torch::TensorOptions& options) {
        if (!workspace_.defined() || static_cast<size_t>(workspace_.numel()) < bytes || workspace_stream_ != stream) {
            workspace_ = torch::empty({static_cast<int64_t>(bytes)}, options);
            workspace_stream_ = stream;
        }
        return workspace_;
    }

    // The stream for calls with a compute-unit budget below the whole device (the reference sizes its
    // cooperative grids with num_sms, csrc/pipeline.cu:20-24, so that communication kernels leave
    // compute units to the caller's own kernels; these kernels are sized by the work, so the budget
    // is enforced where the hardware offers it: a stream created with a CU mask).  Returns the raw
    // handle of a stream whose kernels run on about `cus` compute units, the same number on every
    // XCD; 0 when the budget is the whole device or the device's shape does not allow an even mask.
    // The streams are made on first use, shared by all runtimes of the process and never destroyed:
    // the caching allocator remembers the streams a block was used on and visits them when the block
    // is freed, which may be long after the buffer that used them is closed.
    //
    // Which mask bit is which CU differs between descriptions of the interface (bit i on XCD i mod N,
    // or XCDs one after the other), so the mask is one that gives every XCD the same number of CUs
    // under both readings: with N XCDs of P CUs, bit P*a + N*b + c is set when (a + c) mod N < t.
    // That confines the budget to steps of P (32 of 256 on an MI355X), rounded down, at least one step.
    int64_t budget_stream(int cus) {
        TORCH_CHECK(!closed_.load(), "PeerRuntime is closed");
        int device_cus = 0, xcds = 0;
        check_status(nanoep_device_topology(&device_cus, &xcds, nullptr), "device_topology");
        if (cus <= 0 || cus >= device_cus || xcds <= 1 || device_cus % xcds != 0 || (device_cus / xcds) % xcds != 0)
            return 0;
        const int per_xcd = device_cus / xcds;
        const int steps = std::max(1, cus / per_xcd);  // of `per_xcd` CUs each: per_xcd / xcds on every XCD
        if (steps >= xcds)
            return 0;
        static std::mutex streams_mutex;
        static std::vector<std::tuple<int, int, hipStream_t>> streams;  // (device, steps, stream)
        std::lock_guard<std::mutex> lock(streams_mutex);
        for (const auto& made : streams)
            if (std::get<0>(made) == device_ && std::get<1>(made) == steps)
                return reinterpret_cast<int64_t>(std::get<2>(made));
        std::vector<uint32_t> mask((device_cus + 31) / 32, 0u);
        for (int bit = 0; bit < device_cus; ++bit) {
            const int a = bit / per_xcd, c = bit % xcds;
            if ((a + c) % xcds < steps)
                mask[bit / 32] |= 1u << (bit % 32);
        }
        DeviceGuard guard(static_cast<c10::DeviceIndex>(device_));
        hipStream_t stream = nullptr;
        check_hip(hipExtStreamCreateWithCUMask(&stream, static_cast<uint32_t>(mask.size()), mask.data()), "hipExtStreamCreateWithCUMask");
        streams.emplace_back(device_, steps, stream);
        return reinterpret_cast<int64_t>(stream);
    }

    // compute units a budget stream's kernels can run on (what budget_stream rounds `cus` to)
    int budget_stream_cus(int cus) const {
        int device_cus = 0, xcds = 0;
        check_status(nanoep_device_topology(&device_cus, &xcds, nullptr), "device_topology");
        if (cus <= 0 || cus >= device_cus || xcds <= 1 || device_cus % xcds != 0 || (device_cus / xcds) % xcds != 0)
            return device_cus;
        const int per_xcd = device_cus / xcds;
        const int steps = std::max(1, cus / per_xcd);
        return steps >= xcds ? device_cus : steps * per_xcd;
    }

    py::bytes export_local_handle() const {
        std::string tag(64, '\0');
        tag.replace(0, 9, "nanoep-r1");
        return py::bytes(tag);
    }

    void import_peer_handles(const std::vector<py::bytes>& handles) {
        TORCH_CHECK(!closed_.load(), "PeerRuntime is closed");
        if (handles.size() != 1)
            throw py::value_error("expected exactly one handle (world_size == 1)");
        for (const auto& handle : handles)
            if (py::len(handle) != 64)
                throw py::value_error("Each IPC handle must contain exactly 64 bytes");
        mappings_closed_ = false;
    }

    torch::Tensor local_window() {
        TORCH_CHECK(!closed_.load(), "PeerRuntime is closed");
        if (!window_.defined()) {
            DeviceGuard guard(static_cast<c10::DeviceIndex>(device_));
            window_ = torch::zeros({num_bytes_}, torch::dtype(torch::kUInt8).device(torch::kCUDA, device_));
        }
        return window_;
    }

    torch::Tensor peer_addresses() {
        auto window = local_window();
        auto addresses = torch::empty({1}, torch::dtype(torch::kInt64));
        addresses[0] = reinterpret_cast<int64_t>(window.data_ptr());
        return addresses.to(window.device());
    }

    // No peers: an epoch barrier has nobody to meet.  Epochs still have to increase, as in the
    // reference (csrc/peer.cu:234-237).
    void barrier(int64_t) {
        require_usable();
        ++last_barrier_epoch_;
    }
    void barrier_at(int64_t, int64_t epoch) {
        require_usable();
        TORCH_CHECK(epoch > last_barrier_epoch_, "Barrier epoch must strictly increase");
        last_barrier_epoch_ = epoch;
    }

    void close_peer_mappings() {
        if (closed_.load() || mappings_closed_)
            return;
        TORCH_CHECK(!counts_pending_.load(), "Cannot close while a fresh dispatch is waiting for counts");
        mappings_closed_ = true;
    }

    void close() {
        if (closed_.load())
            return;
        TORCH_CHECK(mappings_closed_, "Call close_peer_mappings() before close()");
        window_ = torch::Tensor();
        forget_private();

        {
            std::lock_guard<std::mutex> lock(counts_mutex_);
            workspace_ = torch::Tensor();
        }
        closed_.store(true);
    }

   private:
    struct RememberedHandle {
        std::optional<c10::weak_intrusive_ptr<c10::TensorImpl>> snapshot;
        uint32_t version = 0;
        const void* snapshot_data = nullptr;
        const void* metadata_data = nullptr;
        int64_t rows = 0;
        int64_t alignment = 0;
        torch::Tensor table, order;
    };

    // in-place edits through torch bump the version; inference tensors have none
    static uint32_t tensor_version(const torch::Tensor& tensor) {
        return tensor.is_inference() ? 0u : tensor.unsafeGetTensorImpl()->version_counter().current_version();
    }

    int device_ = 0;
    int64_t num_bytes_ = 0;
    int64_t* host_counts_ = nullptr;
    torch::Tensor window_;
    std::mutex counts_mutex_;
    std::atomic<bool> counts_pending_{false};
    std::atomic<bool> counts_failed_{false};
    std::atomic<bool> prefers_exact_outputs_{false};
    OutputForecast forecast_;
    std::atomic<int64_t> valid_share_65536_{65536};
    std::deque<RememberedHandle> remembered_;  // newest first
    std::array<std::shared_ptr<RebuiltHandle>, kRebuiltHandles> rebuilt_;
    int64_t* rebuilt_counts_ = nullptr;  // pinned, one word per entry of rebuilt_
    size_t next_rebuilt_ = 0;
    int64_t rebuilt_generation_ = 0;
    int64_t rebuilds_ = 0;
    torch::Tensor workspace_;
    hipStream_t workspace_stream_ = nullptr;
    mutable int64_t private_recalls_ = 0;
    mutable std::mutex private_mutex_;
    int64_t last_barrier_epoch_ = 0;
    bool mappings_closed_ = false;
    std::atomic<bool> closed_{false};
};

// What a caller gets back from an asynchronous call: a marker on the communication stream behind
// the call's kernels, and the tensors those kernels write.  Waiting puts the consumer's stream
// behind the marker and tells the caching allocator that the tensors are in use there, so that
// freeing them on the consumer's side cannot hand their memory out while that stream still reads
// it (the role of csrc/include/nano_ep/event.hpp:12-28 in the reference).
class CompletionEvent {
   public:
    static std::shared_ptr<CompletionEvent> record_behind(const Stream& producer, std::vector<torch::Tensor> written) {
        auto marker = std::make_shared<CompletionEvent>();
        marker->written_ = std::move(written);
        marker->done_.record(producer.unwrap());
        return marker;
    }

    void order_after(const Stream& consumer) const {
        consumer.unwrap().wait(done_);
        for (const auto& tensor : written_)
            if (tensor.defined() && tensor.numel() > 0)
                tensor.record_stream(consumer.unwrap());
    }

    void current_stream_wait() const { order_after(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA()); }

    CompletionEvent() : done_(c10::DeviceType::CUDA) {}

   private:
    c10::Event done_;
    std::vector<torch::Tensor> written_;
};

namespace {

// What a tensor argument has to look like: where it lives, its element type and its extents
// (-1 leaves an extent open).  Every tensor check of dispatch, combine and the cached handle is one
// `require` against such a description; the message is the caller-visible part.
struct TensorSpec {
    c10::Device device;
    at::ScalarType dtype;
    std::vector<int64_t> extents;

    bool describes(const torch::Tensor& tensor) const {
        if (!tensor.defined() || tensor.device() != device || tensor.scalar_type() != dtype || !tensor.is_contiguous() ||
            tensor.dim() != static_cast<int64_t>(extents.size()))
            return false;
        for (size_t axis = 0; axis < extents.size(); ++axis)
            if (extents[axis] >= 0 && tensor.size(static_cast<int64_t>(axis)) != extents[axis])
                return false;
        return true;
    }
};

template <class... Message>
void require(const torch::Tensor& tensor, const TensorSpec& spec, const Message&... message) {
    TORCH_CHECK(spec.describes(tensor), message...);
}

bool vector_aligned(const torch::Tensor& tensor) {
    return tensor.numel() == 0 || reinterpret_cast<uintptr_t>(tensor.data_ptr()) % 16 == 0;
}

// The payload, its routing ids and its weights, as the reference's host pipeline insists on them
// (csrc/pipeline.cu:26-60): same limits, same wording of what is wrong.
void require_dispatch_inputs(const torch::Tensor& x, const torch::Tensor& routing, const c10::optional<torch::Tensor>& weights,
                             int device, int64_t num_experts, int64_t max_tokens) {
    const c10::Device here(c10::DeviceType::CUDA, static_cast<c10::DeviceIndex>(device));
    TORCH_CHECK(x.defined() && x.is_cuda() && x.device() == here && x.dim() == 2 && x.is_contiguous(),
                "x must be contiguous CUDA [T,H] on the runtime device");
    require(x, {here, torch::kBFloat16, {-1, -1}}, "dispatch x must be bfloat16");
    const int64_t tokens = x.size(0), hidden = x.size(1);
    TORCH_CHECK(hidden > 0 && hidden % kHiddenAlignment == 0, "dispatch hidden must be a positive multiple of 256");
    TORCH_CHECK(vector_aligned(x), "dispatch x data pointer must be 16-byte aligned");
    require(routing, {here, torch::kInt64, {tokens, -1}}, "indices must be contiguous CUDA int64 [T,K] on the x device");
    const int64_t topk = routing.size(1);
    TORCH_CHECK(topk >= 1 && topk <= 32, "num_topk must be in [1, 32]");
    TORCH_CHECK(num_experts > 0, "num_experts must be positive and divisible by world_size");
    TORCH_CHECK(max_tokens <= std::numeric_limits<int32_t>::max(), "max_tokens exceeds int32 metadata range");
    TORCH_CHECK(max_tokens > 0 && tokens <= max_tokens, "source token count exceeds max_tokens");
    if (weights.has_value())
        require(*weights, {here, torch::kFloat32, {tokens, topk}}, "weights must be contiguous CUDA float32 [T,K] on the x device");
}

// The seven handle tensors of a cached call against the geometry they must describe.
void require_handle_tensors(const std::vector<torch::Tensor>& metadata, const c10::Device& here, int64_t source_tokens, int64_t topk,
                            int64_t local_experts) {
    struct Field {
        const char* name;
        at::ScalarType dtype;
        std::vector<int64_t> extents;
    };
    const Field fields[7] = {
        {"recv_metadata", torch::kInt32, {-1, topk + 2}},
        {"expert_counts", torch::kInt64, {local_experts}},
        {"expert_offsets", torch::kInt64, {local_experts + 1}},
        {"dst_slots", torch::kInt64, {source_tokens, 1}},
        {"send_counts", torch::kInt64, {1}},
        {"source_topk_snapshot", torch::kInt64, {source_tokens, topk}},
        {"recv_rank_prefix", torch::kInt64, {1}},
    };
    for (int i = 0; i < 7; ++i)
        require(metadata[i], {here, fields[i].dtype, fields[i].extents}, "cached ", fields[i].name, " has invalid CUDA storage or shape");
}

// The optional eighth handle tensor: int32 [T,K] slot table written by the layout kernels.
const int32_t* slot_table(const std::vector<torch::Tensor>& metadata, int64_t tokens, int64_t topk, bool expand) {
    if (!expand || metadata.size() < 8 || !metadata[7].defined())
        return nullptr;
    const auto& table = metadata[7];
    TORCH_CHECK(table.device() == metadata[0].device() && table.scalar_type() == torch::kInt32 && table.is_contiguous() &&
                    table.dim() == 2 && table.size(0) == tokens && table.size(1) == topk,
                "cached slot table has invalid CUDA storage or shape");
    return table.numel() == 0 ? nullptr : table.data_ptr<int32_t>();
}

// The optional ninth handle tensor: int64 slot-order list written by the layout kernels.
const int64_t* slot_order_list(const std::vector<torch::Tensor>& metadata, int64_t tokens, int64_t topk, int64_t local_experts,
                               bool expand, int64_t* entries) {
    *entries = 0;
    if (!expand || metadata.size() < 9 || !metadata[8].defined())
        return nullptr;
    const auto& order = metadata[8];
    TORCH_CHECK(order.device() == metadata[0].device() && order.scalar_type() == torch::kInt64 && order.is_contiguous() &&
                    order.dim() == 1 && order.size(0) <= nanoep_slot_order_entries(tokens, static_cast<int>(topk), local_experts),
                "cached slot-order list has invalid CUDA storage or shape");
    // the whole buffer (list + count word) defers to the count on the device
    const bool whole = order.numel() > 0 && order.numel() == nanoep_slot_order_entries(tokens, static_cast<int>(topk), local_experts);
    *entries = whole ? -1 : order.numel();
    return order.numel() == 0 ? nullptr : order.data_ptr<int64_t>();
}

// Communication stream waits for the producer of the inputs: the caller's stream, an explicit
// event, or both (csrc/pipeline.cu:364-377 in the reference).
// An external-stream wrapper never compares equal to a pool stream object, so identity is decided
// on the raw handles: when the caller already runs on the communication stream no event is needed.
bool same_queue(const Stream& a, const Stream& b) { return a.stream() == b.stream(); }

// Stream the kernels are enqueued on.  An asynchronous call uses the buffer's communication stream.
// A synchronous call must leave its results ordered on the caller's stream, so it runs there
// directly instead of bouncing through the communication stream with two cross-stream events; it
// still comes after everything enqueued earlier on the communication stream.
Stream work_stream(int64_t comm_handle, const Stream& compute, c10::DeviceIndex device, bool async_op, bool budgeted) {
    const auto comm = external_stream(comm_handle, device);
    // (a call with a compute-unit budget runs on the stream it was handed: that stream carries the CU mask)
    if (async_op || budgeted || same_queue(comm, compute))
        return comm;
    // While the caller's stream is being captured into a graph no other stream may be queried;
    // a captured call is ordered by the graph alone.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    check_hip(hipStreamIsCapturing(compute.stream(), &capture), "hipStreamIsCapturing");
    if (capture == hipStreamCaptureStatusNone && hipStreamQuery(comm.stream()) == hipErrorNotReady)
        wait_on(compute, comm);
    return compute;
}

void order_comm_after_inputs(const Stream& comm, const Stream& compute, int64_t previous_event, bool async_op) {
    if (previous_event != -1) {
        if (!async_op && !same_queue(comm, compute))
            wait_on(comm, compute);
        check_hip(hipStreamWaitEvent(comm.stream(), reinterpret_cast<hipEvent_t>(previous_event), 0), "hipStreamWaitEvent");
    } else if (!same_queue(comm, compute)) {
        wait_on(comm, compute);
    }
}

// The private tensors of a seven-tensor expanded handle the runtime does not remember: found among
// the ones rebuilt earlier, or rebuilt now on `stream` (the current stream of the allocator).
std::shared_ptr<PeerRuntime::RebuiltHandle> private_tensors_of(PeerRuntime& runtime, const std::vector<torch::Tensor>& metadata,
                                                               int64_t capacity, int64_t tokens, int64_t topk, int64_t local_experts,
                                                               int64_t hidden, const Stream& stream) {
    auto entry = runtime.find_rebuilt(metadata, capacity);
    if (entry) {
        if (entry->made_on != stream.stream()) {
            // built on another stream: wait for it unless it is long done, and tell the allocator
            if (!entry->ready.query())
                stream.unwrap().wait(entry->ready);
            entry->order.record_stream(stream.unwrap());  // the table is a view of the same allocation
        }
        return entry;
    }
    entry = runtime.new_rebuilt(metadata, capacity);
    const int64_t order_words = nanoep_slot_order_entries(tokens, static_cast<int>(topk), local_experts);
    const size_t workspace_bytes = nanoep_rebuild_workspace_bytes(tokens, static_cast<int>(topk));
    const int64_t table_words = (tokens * topk + 1) / 2;
    const int64_t workspace_words = static_cast<int64_t>((workspace_bytes + 7) / 8);
    // one allocation: slot-order buffer | slot table | the rebuild's scratch
    auto storage = torch::empty({order_words + table_words + workspace_words}, metadata[3].options());
    entry->order = storage.narrow(0, 0, order_words);
    entry->table = storage.narrow(0, order_words, table_words).view(torch::kInt32).narrow(0, 0, tokens * topk).view({tokens, topk});
    check_status(nanoep_rebuild_order(metadata[0].data_ptr<int32_t>(), metadata[3].data_ptr<int64_t>(), metadata[0].size(0), capacity, tokens,
                                      static_cast<int>(topk), local_experts, static_cast<int>(hidden), entry->table.data_ptr<int32_t>(),
                                      entry->order.data_ptr<int64_t>(), storage.data_ptr<int64_t>() + order_words + table_words,
                                      static_cast<size_t>(workspace_words) * 8, entry->count, entry->tag, stream.stream()),
                 "rebuild_order");
    entry->made_on = stream.stream();
    entry->ready.record(stream.unwrap());
    runtime.publish_rebuilt(entry);
    return entry;
}

}  // namespace

using DispatchResult =
    std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>, std::array<int64_t, 2>, std::shared_ptr<CompletionEvent>>;

DispatchResult dispatch(PeerRuntime& runtime,
                        const torch::Tensor& x,
                        const torch::Tensor& indices,
                        const c10::optional<torch::Tensor>& weights,
                        int64_t num_experts,
                        int64_t max_tokens,
                        int64_t alignment,
                        const std::vector<torch::Tensor>& cached_metadata,
                        int64_t cached_expanded_capacity,
                        bool /*allow_multiple_reduction*/,
                        bool expand,
                        bool zero_padding,
                        int num_sms,
                        int64_t comm_stream,
                        int64_t previous_event,
                        bool async_op) {
    const bool cached = !cached_metadata.empty();
    TORCH_CHECK(!cached || (cached_metadata.size() >= 7 && cached_metadata.size() <= 9),
                "cached metadata must contain the seven prepared tensors from dispatch (plus the optional slot table and slot-order list)");
    const auto& routing = cached ? cached_metadata[5] : indices;
    runtime.require_usable();
    require_dispatch_inputs(x, routing, weights, runtime.device(), num_experts, max_tokens);
    TORCH_CHECK(alignment > 0, "alignment must be positive");
    const auto device = static_cast<c10::DeviceIndex>(runtime.device());
    DeviceGuard device_guard(device);
    const int cu_budget = resolve_cu_budget(num_sms, device);

    const int64_t tokens = x.size(0);
    const int64_t hidden = x.size(1);
    const int64_t topk = routing.size(1);
    const int64_t local_experts = num_experts;

    const auto compute = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device);
    const auto comm = work_stream(comm_stream, compute, device, async_op, cu_budget != 0);
    order_comm_after_inputs(comm, compute, previous_event, async_op);

    StreamGuard comm_guard(comm.unwrap());
    // Sync results belong to the caller's stream, async results to the communication stream
    // (protected by record_stream when the consumer waits on the completion event).
    const auto allocate_for_consumer = [&](auto&& make) {
        OptionalStreamGuard allocation_guard;
        if (!async_op)
            allocation_guard.reset_stream(compute.unwrap());
        return make();
    };

    const auto float_options = x.options().dtype(torch::kFloat32);
    torch::Tensor out_x, out_indices, out_weights;
    // x_rows rows of payload (and expanded weights), n_rows rows of compact indices / weights
    const auto allocate_outputs = [&](int64_t x_rows, int64_t n_rows) {
        allocate_for_consumer([&] {
            out_x = torch::empty({x_rows, hidden}, x.options());
            if (!expand)
                out_indices = torch::empty({n_rows, topk}, routing.options());
            out_weights = !weights.has_value() ? torch::empty({0}, float_options)
                          : expand            ? torch::empty({x_rows}, float_options)
                                              : torch::empty({n_rows, topk}, float_options);
            return 0;
        });
    };
    // What the permute reads of a handle, as plain pointers.  order_entries: A, or -1 for "the whole
    // slot-order buffer is there and the kernel finds A in its last word".
    struct HandleView {
        const int32_t* recv_metadata = nullptr;
        const int64_t* dst_slots = nullptr;
        const int32_t* token_slots = nullptr;
        const int64_t* slot_order = nullptr;
        int64_t order_entries = 0;
        const int64_t* expert_counts = nullptr;
        const int64_t* expert_offsets = nullptr;
    };
    const auto view_of = [&](const std::vector<torch::Tensor>& handle) {
        HandleView view;
        view.recv_metadata = handle[0].data_ptr<int32_t>();
        view.dst_slots = handle[3].data_ptr<int64_t>();
        view.token_slots = slot_table(handle, tokens, topk, expand);
        view.slot_order = slot_order_list(handle, tokens, topk, local_experts, expand, &view.order_entries);
        view.expert_counts = handle[1].data_ptr<int64_t>();
        view.expert_offsets = handle[2].data_ptr<int64_t>();
        return view;
    };
    // count_on_device: the number of list entries in use is not known on the host yet
    const auto launch_permute = [&](HandleView handle, int64_t received, int64_t capacity, bool count_on_device = false) {
        TORCH_CHECK(!count_on_device || handle.slot_order == nullptr || handle.order_entries == -1, "slot-order buffer is incomplete");
        if (count_on_device && handle.slot_order != nullptr) {
            // the launch is sized for the share of valid choices the runtime saw last, plus 0.5 %
            const int64_t share = runtime.valid_share_65536() + 328;
            const int64_t expected = share >= 65536 ? tokens * topk : tokens * topk * share / 65536;
            handle.order_entries = expected >= tokens * topk || expected < 2 ? -1 : -expected;
        }
        check_status(
            nanoep_dispatch(x.data_ptr(), weights.has_value() ? weights->data_ptr<float>() : nullptr, handle.recv_metadata, handle.dst_slots,
                            handle.token_slots, handle.slot_order, handle.order_entries, handle.expert_counts, handle.expert_offsets,
                            received, capacity, tokens, static_cast<int>(hidden), static_cast<int>(topk), local_experts, alignment,
                            expand ? 1 : 0, zero_padding ? 1 : 0, out_x.data_ptr(), expand ? nullptr : out_indices.data_ptr<int64_t>(),
                            weights.has_value() ? out_weights.data_ptr<float>() : nullptr, cu_budget, comm.stream()),
            "dispatch");
    };

    std::vector<torch::Tensor> metadata;
    int64_t recv_count = 0;
    int64_t expanded_capacity = 0;
    if (cached) {
        require_handle_tensors(cached_metadata, x.device(), tokens, topk, local_experts);
        metadata = cached_metadata;
        recv_count = cached_metadata[0].size(0);
        expanded_capacity = cached_expanded_capacity;
        TORCH_CHECK(recv_count <= tokens && expanded_capacity >= 0, "cached handle does not match the payload");
        TORCH_CHECK(!expand || expanded_capacity <= std::numeric_limits<int32_t>::max(),
                    "expanded capacity exceeds int32 metadata range");
        allocate_outputs(expand ? expanded_capacity : recv_count, recv_count);
        // A handle that went through the reference's Python class carries the seven tensors of the
        // reference only.  If it is one of this runtime's latest fresh dispatches, the runtime still
        // has its private tensors and the payload takes the slot-order walk
        // (the RECALL_ORDER switch set to 0 turns that off).  Any other seven-tensor handle is followed as it
        // is written, in token order through its own dst_slots and recv_metadata: whatever row and
        // slot order it describes is the order the rows land in.
        bool has_private = metadata.size() > 7;
        if (expand && recv_count > 0 && !has_private && tuning_switch("RECALL_ORDER") != 0)
            has_private = runtime.recall_private(metadata, alignment);
        if (recv_count > 0) {
            HandleView view = view_of(metadata);
            // A seven-tensor handle the runtime does not remember: its private tensors are rebuilt from
            // the handle as it is written (one integer pass, two launches) and kept for its later
            // replays, where the payload is large enough for the slot-order walk to pay for that
            // (the REBUILD_ORDER switch: 0 never, 1 always).  Not under stream capture: a captured
            // replay must not depend on when the rebuilt tensors are dropped.
            const int rebuild_switch = tuning_switch("REBUILD_ORDER");
            const bool worth_it = rebuild_switch >= 0 ? rebuild_switch != 0 : expanded_capacity * hidden * 2 >= kRebuildPayloadBytes;
            std::shared_ptr<PeerRuntime::RebuiltHandle> rebuilt;
            if (expand && !has_private && worth_it && tokens * topk < (int64_t{1} << 31) &&
                nanoep_slot_order_entries(tokens, static_cast<int>(topk), local_experts) > 0) {
                hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
                check_hip(hipStreamIsCapturing(comm.stream(), &capture), "hipStreamIsCapturing");
                if (capture == hipStreamCaptureStatusNone)
                    rebuilt = private_tensors_of(runtime, metadata, expanded_capacity, tokens, topk, local_experts, hidden, comm);
            }
            if (rebuilt) {
                view.token_slots = rebuilt->table.data_ptr<int32_t>();
                view.slot_order = rebuilt->order.data_ptr<int64_t>();
                const int64_t entries = rebuilt->published_entries();
                view.order_entries = entries >= 0 ? entries : -1;
            }
            launch_permute(view, recv_count, expanded_capacity, /*count_on_device=*/rebuilt && view.order_entries < 0);
        }
    } else {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        check_hip(hipStreamIsCapturing(comm.stream(), &capture), "hipStreamIsCapturing");
        TORCH_CHECK(capture == hipStreamCaptureStatusNone, "Fresh dispatch with host count polling cannot be captured in a HIP graph");

        const auto int64_options = routing.options();
        torch::Tensor recv_metadata, expert_counts, expert_offsets, dst_slots, send_counts, snapshot, prefix, token_slots, slot_order;
        // the slot-order list packs token * K + k into 32 bits
        const bool ordered = expand && tokens * topk < (int64_t{1} << 31);
        // The handle tensors of one call are views of one allocation (the int64 ones, then the int32 ones), and the
        // views are made after the layout has been enqueued: on a path whose small-batch cost is
        // host latency, the GPU starts three allocator round trips after the call instead of ten
        // and works while the rest of the bookkeeping is done.
        const int64_t order_entries = ordered ? nanoep_slot_order_entries(tokens, static_cast<int>(topk), local_experts) : 0;
        // offsets of the int64 tensors in the arena; the per-token ones start 16-byte aligned (even
        // offsets), which lets the layout kernels move two ids a lane at a time
        const auto even = [](int64_t words) { return (words + 1) / 2 * 2; };
        const int64_t at_offsets = local_experts, at_send = 2 * local_experts + 1, at_prefix = at_send + 1;
        const int64_t at_dst = even(at_prefix + 1), at_snapshot = even(at_dst + tokens), at_order = even(at_snapshot + tokens * topk);
        const int64_t count64 = even(at_order + order_entries);
        const int64_t at_table = (tokens * (topk + 2) + 3) / 4 * 4;  // the slot table starts 16-byte aligned
        const int64_t count32 = at_table + (expand ? tokens * topk : 0);
        const size_t workspace_bytes = nanoep_layout_workspace_bytes(tokens, static_cast<int>(topk), local_experts);
        TORCH_CHECK(workspace_bytes > 0, "unsupported routing geometry for the layout kernels");
        TORCH_CHECK(nanoep_layout_block_tokens(tokens, local_experts, static_cast<int>(hidden)) > 0,
                    "the layout kernels take at most 3839 local experts, got ", local_experts);
        // one allocation: the int64 tensors first, the int32 ones behind them as a view of the same storage
        torch::Tensor arena64, arena32;
        allocate_for_consumer([&] {
            arena64 = torch::empty({count64 + (count32 + 1) / 2}, int64_options);
            return 0;
        });
        // arena64: expert_counts [L] | expert_offsets [L+1] | send_counts [1] | recv_rank_prefix [1] |
        //          dst_slots [T] | topk snapshot [T*K] | slot_order;   arena32: recv_metadata [T*(K+2)] | token_slots [T*K]
        int64_t* base64 = arena64.data_ptr<int64_t>();
        int32_t* base32 = reinterpret_cast<int32_t*>(base64 + count64);

        // From here until the counts have been read this call owns the runtime's mailbox; a fresh
        // dispatch of another thread on the same runtime waits here for its turn.
        PeerRuntime::CountsTurn turn(runtime);
        const auto workspace = runtime.layout_workspace(workspace_bytes, comm.stream(), int64_options.dtype(torch::kUInt8));
        const int layout_status =
            nanoep_layout(routing.data_ptr<int64_t>(), tokens, static_cast<int>(topk), local_experts, alignment, expand ? 1 : 0,
                          static_cast<int>(hidden), base32, base64, base64 + at_offsets, base64 + at_dst, base64 + at_send, base64 + at_snapshot,
                          base64 + at_prefix, expand ? base32 + at_table : nullptr, order_entries > 0 ? base64 + at_order : nullptr,
                          workspace.data_ptr(), workspace_bytes, turn.mailbox(), comm.stream());
        if (layout_status != NANOEP_OK && layout_status != NANOEP_ERR_HIP)
            turn.abandon();  // refused before anything was enqueued
        check_status(layout_status, "layout");

        // The exact shapes (N, C) are only known once the layout kernels have run.  Waiting for
        // them before launching the permute leaves the GPU idle for a host round trip, so where the
        // upper bound of the shapes (every choice valid plus every expert's worst alignment gap) is
        // close to what routing will fill, the outputs are allocated at that bound, the permute is
        // enqueued right behind the layout and the results are narrowed afterwards.  "Close" is
        // kept honest in both directions: the gaps may add at most an eighth to the bound, and a call
        // that still ends up holding more than 1.25 times the rows it uses (many masked choices)
        // permutes again into exact outputs and turns the runtime to the exact order, in which the
        // outputs are allocated after the counts are known, until a call shows the bound close again.
        const int64_t choice_bound = expand ? tokens * topk : tokens;
        const int64_t gap_bound = expand ? local_experts * (alignment - 1) : 0;
        const int64_t row_bound = choice_bound + gap_bound;
        const int order_switch = tuning_switch("FRESH_OUTPUTS");  // 0: always exact, 1: at the bound whenever the rule allows it
        const bool bound_rule = gap_bound * 8 <= choice_bound;
        PeerRuntime::OutputForecast geometry;
        geometry.tokens = tokens, geometry.topk = topk, geometry.experts = local_experts, geometry.alignment = alignment;
        geometry.hidden = hidden, geometry.expand = expand;
        // rows the outputs are allocated for ahead of the counts: the bound where it is close, else what
        // the latest call of this geometry used plus an eighth, else nothing (the exact order)
        int64_t early_rows = 0;
        if (tokens > 0 && order_switch != 0 && row_bound <= std::numeric_limits<int32_t>::max()) {
            if (bound_rule && (order_switch == 1 || !runtime.prefers_exact_outputs()))
                early_rows = row_bound;
            else if (!bound_rule)
                early_rows = std::min(row_bound, runtime.forecast_rows(geometry));
        }
        const bool speculative = early_rows > 0;
        if (speculative) {
            // enqueued straight from the arena's pointers: the tensors of the handle are made below,
            // while the GPU works
            HandleView fresh;
            fresh.recv_metadata = base32;
            fresh.dst_slots = base64 + at_dst;
            fresh.token_slots = expand ? base32 + at_table : nullptr;
            fresh.slot_order = order_entries > 0 ? base64 + at_order : nullptr;
            fresh.order_entries = order_entries > 0 ? -1 : 0;
            fresh.expert_counts = base64;
            fresh.expert_offsets = base64 + at_offsets;
            try {
                allocate_outputs(early_rows, tokens);
                launch_permute(fresh, tokens, early_rows, /*count_on_device=*/true);
            } catch (...) {
                // The layout is under way and will publish its counts whatever went wrong here (most
                // likely the allocation at the bound): the turn at the mailbox is settled before the
                // error leaves, so the runtime stays usable.  Only counts that never arrive latch it.
                int64_t unused[NANOEP_HOST_COUNT_WORDS] = {0, 0, 0, 0};
                try {
                    turn.wait(comm.stream(), kCountTimeoutSeconds, unused);
                } catch (...) {
                }
                throw;
            }
        }

        arena32 = arena64.narrow(0, count64, (count32 + 1) / 2).view(torch::kInt32);
        expert_counts = arena64.narrow(0, 0, local_experts);
        expert_offsets = arena64.narrow(0, at_offsets, local_experts + 1);
        send_counts = arena64.narrow(0, at_send, 1);
        prefix = arena64.narrow(0, at_prefix, 1);
        dst_slots = arena64.narrow(0, at_dst, tokens).view({tokens, 1});
        snapshot = arena64.narrow(0, at_snapshot, tokens * topk).view({tokens, topk});
        recv_metadata = arena32.narrow(0, 0, tokens * (topk + 2)).view({tokens, topk + 2});
        metadata = {recv_metadata, expert_counts, expert_offsets, dst_slots, send_counts, snapshot, prefix};
        if (expand) {
            token_slots = arena32.narrow(0, at_table, tokens * topk).view({tokens, topk});
            metadata.push_back(token_slots);  // private eighth entry: slot[t,k] in one lookup
        }
        if (ordered) {
            slot_order = arena64.narrow(0, at_order, order_entries);
            metadata.push_back(slot_order);  // private ninth entry: assignments in block-wise slot order
        }

        int64_t counts[NANOEP_HOST_COUNT_WORDS] = {0, 0, 0, 0};
        const int status = turn.wait(comm.stream(), kCountTimeoutSeconds, counts);
        if (status == NANOEP_ERR_ROUTING) {
            TORCH_CHECK(false, "dispatch routing ids must be -1 or distinct expert ids in [0, ", local_experts, ")",
                        (counts[3] & NANOEP_ROUTING_BAD_EXPERT) ? "; found an id out of range" : "",
                        (counts[3] & NANOEP_ROUTING_DUPLICATE) ? "; found a duplicate expert within a token" : "");
        }
        recv_count = counts[0];
        expanded_capacity = counts[1];
        TORCH_CHECK(recv_count >= 0 && recv_count <= tokens, "dispatch receive count exceeds the source token count");
        TORCH_CHECK(!expand || expanded_capacity <= std::numeric_limits<int32_t>::max(),
                    "expanded capacity exceeds int32 metadata range");
        metadata[0] = recv_metadata.narrow(0, 0, recv_count);
        if (ordered) {
            TORCH_CHECK(counts[2] >= 0 && counts[2] <= slot_order.size(0), "assignment count exceeds the slot-order list");
            metadata[8] = slot_order.narrow(0, 0, counts[2]);  // replays walk the A assignments only
            runtime.note_valid_share(counts[2], tokens * topk);
        }
        const int64_t used_rows = expand ? expanded_capacity : recv_count;
        const bool bound_is_close = used_rows * 5 >= row_bound * 4;  // the bound holds at most 1.25 x the rows in use
        TORCH_CHECK(used_rows <= row_bound, "receive rows exceed their upper bound");
        // the early outputs are kept when every row in use has a place in them and they hold at most 1.25 x those rows
        const bool early_outputs_fit = speculative && used_rows <= early_rows && used_rows * 5 >= early_rows * 4;
        runtime.note_used_rows(geometry, used_rows);
        if (early_outputs_fit) {
            out_x = out_x.narrow(0, 0, used_rows);
            if (!expand)
                out_indices = out_indices.narrow(0, 0, recv_count);
            if (weights.has_value())
                out_weights = out_weights.narrow(0, 0, used_rows);
        } else {
            allocate_outputs(used_rows, recv_count);
            if (recv_count > 0)
                launch_permute(view_of(metadata), recv_count, expanded_capacity);
        }
        if (tokens > 0 && bound_rule)
            runtime.note_output_fill(bound_is_close);
        if (expand)
            runtime.remember_private(metadata, alignment);
    }

    if (expand)
        out_indices = torch::empty({0}, routing.options());  // absent at this boundary; made off the path to the launch
    std::vector<torch::Tensor> outputs{out_x, out_indices, out_weights};
    std::shared_ptr<CompletionEvent> event;
    if (async_op) {
        if (x.numel() > 0)
            x.record_stream(comm.unwrap());
        if (!cached && indices.numel() > 0)
            indices.record_stream(comm.unwrap());
        if (weights.has_value() && weights->numel() > 0)
            weights->record_stream(comm.unwrap());
        for (const auto& tensor : cached_metadata)
            if (tensor.numel() > 0)
                tensor.record_stream(comm.unwrap());
        auto protected_tensors = outputs;
        protected_tensors.insert(protected_tensors.end(), metadata.begin(), metadata.end());
        event = CompletionEvent::record_behind(comm, std::move(protected_tensors));
    } else if (!same_queue(comm, compute)) {
        wait_on(compute, comm);
    }
    return std::make_tuple(std::move(outputs), std::move(metadata), std::array<int64_t, 2>{recv_count, expanded_capacity}, std::move(event));
}

using CombineResult = std::tuple<std::vector<torch::Tensor>, std::shared_ptr<CompletionEvent>>;

CombineResult combine(PeerRuntime& runtime,
                      const torch::Tensor& x,
                      const std::vector<torch::Tensor>& metadata,
                      const c10::optional<torch::Tensor>& weights,
                      const c10::optional<torch::Tensor>& bias,
                      int64_t max_tokens,
                      bool expand,
                      bool allow_multiple_reduction,
                      int num_sms,
                      int64_t comm_stream,
                      int64_t previous_event,
                      bool async_op) {
    TORCH_CHECK(metadata.size() >= 7 && metadata.size() <= 9 && x.defined() && x.dim() == 2 && metadata[5].dim() == 2,
                "combine requires a 2D payload and seven prepared metadata tensors");
    runtime.require_usable();
    const auto device = static_cast<c10::DeviceIndex>(runtime.device());
    DeviceGuard device_guard(device);
    const c10::Device here(c10::DeviceType::CUDA, device);
    TORCH_CHECK(x.is_cuda() && x.device() == here && x.is_contiguous() && x.size(1) > 0,
                "combine x must be contiguous CUDA [N,H] or [C,H] on the runtime device");
    require(x, {here, torch::kBFloat16, {-1, -1}}, "combine x must be bfloat16");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0, "combine x data pointer must be 16-byte aligned");
    TORCH_CHECK(x.size(1) % kHiddenAlignment == 0, "combine hidden must be a positive multiple of 256");
    TORCH_CHECK(metadata[1].dim() == 1 && metadata[1].numel() > 0,
                "combine metadata requires a [T,K] source snapshot and [L] expert counts");

    const int64_t recv_count = metadata[0].dim() == 2 ? metadata[0].size(0) : -1;
    const int64_t source_tokens = metadata[5].size(0);
    const int64_t hidden = x.size(1);
    const int64_t topk = metadata[5].size(1);
    const int64_t local_experts = metadata[1].numel();
    TORCH_CHECK(topk > 0 && topk <= 32 && topk <= local_experts && source_tokens <= max_tokens && recv_count <= max_tokens,
                "combine routing geometry exceeds expert/token capacity");
    require_handle_tensors(metadata, here, source_tokens, topk, local_experts);
    TORCH_CHECK(expand ? (x.size(0) >= recv_count && (recv_count != 0 || x.size(0) == 0)) : x.size(0) == recv_count,
                "combine x rows do not match the receive layout");
    if (weights.has_value())
        require(*weights, {here, torch::kFloat32, expand ? std::vector<int64_t>{x.size(0)} : std::vector<int64_t>{recv_count, topk}},
                "combine weights must be contiguous CUDA float32 [N,K] or expanded [C] on the x device");
    if (bias.has_value())
        require(*bias, {here, torch::kBFloat16, {source_tokens, hidden}},
                "combine bias must be contiguous [T,H], with the output dtype on the x device");
    const int cu_budget = resolve_cu_budget(num_sms, device);

    const auto compute = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device);
    const auto comm = work_stream(comm_stream, compute, device, async_op, cu_budget != 0);
    order_comm_after_inputs(comm, compute, previous_event, async_op);
    StreamGuard comm_guard(comm.unwrap());

    torch::Tensor combined_x, combined_weights;
    {
        OptionalStreamGuard allocation_guard;
        if (!async_op)
            allocation_guard.reset_stream(compute.unwrap());
        combined_x = torch::empty({source_tokens, hidden}, x.options());
        combined_weights = torch::empty(weights.has_value() ? std::vector<int64_t>{source_tokens, topk} : std::vector<int64_t>{0},
                                        x.options().dtype(torch::kFloat32));
    }
    if (source_tokens > 0) {
        // a seven-tensor handle of the latest fresh dispatch gets its slot table back from the runtime
        std::vector<torch::Tensor> handle;
        if (expand && metadata.size() == 7 && tuning_switch("RECALL_ORDER") != 0) {
            handle = metadata;
            runtime.recall_private(handle, -1);
        }
        const auto& lookup = handle.size() > 7 ? handle : metadata;
        const int32_t* table = slot_table(lookup, source_tokens, topk, expand);
        // ... or the table a replayed dispatch of this handle had rebuilt
        std::shared_ptr<PeerRuntime::RebuiltHandle> rebuilt;
        if (table == nullptr && expand && metadata.size() == 7 && recv_count > 0 && tuning_switch("REBUILD_ORDER") != 0) {
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            check_hip(hipStreamIsCapturing(comm.stream(), &capture), "hipStreamIsCapturing");
            if (capture == hipStreamCaptureStatusNone && (rebuilt = runtime.find_rebuilt(metadata, x.size(0)))) {
                if (rebuilt->made_on != comm.stream()) {
                    if (!rebuilt->ready.query())
                        comm.unwrap().wait(rebuilt->ready);
                    rebuilt->order.record_stream(comm.unwrap());
                }
                table = rebuilt->table.data_ptr<int32_t>();
            }
        }
        check_status(nanoep_combine(x.data_ptr(), weights.has_value() ? weights->data_ptr<float>() : nullptr,
                                    bias.has_value() ? bias->data_ptr() : nullptr, metadata[0].data_ptr<int32_t>(),
                                    metadata[3].data_ptr<int64_t>(), table, recv_count,
                                    x.size(0), source_tokens, static_cast<int>(hidden),
                                    static_cast<int>(topk), expand ? 1 : 0, allow_multiple_reduction ? 1 : 0, combined_x.data_ptr(),
                                    weights.has_value() ? combined_weights.data_ptr<float>() : nullptr, cu_budget, comm.stream()),
                     "combine");
    }

    std::vector<torch::Tensor> outputs{combined_x, combined_weights};
    std::shared_ptr<CompletionEvent> event;
    if (async_op) {
        if (x.numel() > 0)
            x.record_stream(comm.unwrap());
        if (weights.has_value() && weights->numel() > 0)
            weights->record_stream(comm.unwrap());
        if (bias.has_value() && bias->numel() > 0)
            bias->record_stream(comm.unwrap());
        for (const auto& tensor : metadata)
            if (tensor.numel() > 0)
                tensor.record_stream(comm.unwrap());
        event = CompletionEvent::record_behind(comm, outputs);
    } else if (!same_queue(comm, compute)) {
        wait_on(compute, comm);
    }
    return std::make_tuple(std::move(outputs), std::move(event));
}

std::vector<int64_t> window_layout(int ranks, int64_t tokens, int hidden, int topk, int64_t num_experts, bool allow_multiple_reduction) {
    int64_t out[5] = {0, 0, 0, 0, 0};
    const int status = nanoep_window_layout(ranks, tokens, hidden, topk, num_experts, allow_multiple_reduction ? 1 : 0, out);
    if (status != NANOEP_OK)
        throw py::value_error("window_layout requires ranks/topk in [1,32], positive capacity/hidden and num_experts divisible by ranks");
    return {out[0], out[1], out[2], out[3], out[4]};
}

}  // namespace nanoep

PYBIND11_MODULE(TORCH_EXTENSION_NAME, module) {
    module.doc() = "MI355X dispatch / combine host extension (ahead-of-time HIP kernels behind a C ABI)";
    module.attr("abi_version") = nanoep_abi_version();
    // Kernels are compiled ahead of time: the JIT warm-up entry points are accepted and ignored.
    module.def("init_jit", [](const std::string&) {});
    module.def("prepare_dispatch", [](py::args, py::kwargs) {});
    module.def("prepare_combine", [](py::args, py::kwargs) {});
    module.def("dispatch", &nanoep::dispatch, py::arg("runtime"), py::arg("x"), py::arg("indices"), py::arg("weights"),
               py::arg("num_experts"), py::arg("max_tokens"), py::arg("alignment"), py::arg("cached_metadata"),
               py::arg("cached_expanded_capacity"), py::arg("allow_multiple_reduction"), py::arg("expand"), py::arg("zero_padding"),
               py::arg("num_sms"), py::arg("comm_stream"), py::arg("previous_event") = -1, py::arg("async_op") = true,
               py::call_guard<py::gil_scoped_release>());
    module.def("combine", &nanoep::combine, py::arg("runtime"), py::arg("x"), py::arg("metadata"), py::arg("weights"), py::arg("bias"),
               py::arg("max_tokens"), py::arg("expand"), py::arg("allow_multiple_reduction"), py::arg("num_sms"), py::arg("comm_stream"),
               py::arg("previous_event") = -1, py::arg("async_op") = true, py::call_guard<py::gil_scoped_release>());
    module.def("window_layout", &nanoep::window_layout, py::arg("ranks"), py::arg("tokens"), py::arg("hidden"), py::arg("topk"),
               py::arg("num_experts"), py::arg("allow_multiple_reduction") = false);
    py::class_<nanoep::PeerRuntime>(module, "PeerRuntime")
        .def(py::init<int, int, int64_t>())
        .def("export_local_handle", &nanoep::PeerRuntime::export_local_handle)
        .def("import_peer_handles", &nanoep::PeerRuntime::import_peer_handles)
        .def("peer_addresses", &nanoep::PeerRuntime::peer_addresses)
        .def("local_window", &nanoep::PeerRuntime::local_window)
        .def("barrier", &nanoep::PeerRuntime::barrier)
        .def("barrier", &nanoep::PeerRuntime::barrier_at)
        .def("close_peer_mappings", &nanoep::PeerRuntime::close_peer_mappings)
        .def("private_recalls", &nanoep::PeerRuntime::private_recalls)
        .def("rebuilds", &nanoep::PeerRuntime::rebuilds)
        .def("budget_stream", &nanoep::PeerRuntime::budget_stream)
        .def("budget_stream_cus", &nanoep::PeerRuntime::budget_stream_cus)
        .def("counts_failed", &nanoep::PeerRuntime::counts_failed)
        .def("prefers_exact_outputs", &nanoep::PeerRuntime::prefers_exact_outputs)
        .def("valid_share_65536", &nanoep::PeerRuntime::valid_share_65536)
        .def("lose_counts_for_test", &nanoep::PeerRuntime::lose_counts_for_test)
        .def("close", &nanoep::PeerRuntime::close);
    py::class_<nanoep::CompletionEvent, std::shared_ptr<nanoep::CompletionEvent>>(module, "CompletionEvent")
        .def("current_stream_wait", &nanoep::CompletionEvent::current_stream_wait);
}
