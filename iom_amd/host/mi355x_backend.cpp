// MI355X backend for IOM: iom::Device / iom::Tensor / iom::RawWorkspace /
// iom::DeviceOps subclasses behind the factory iom::make_rocm_device
// (include/iom/rocm/device.hpp:22-24), a drop-in for the reference's ROCm
// backend on the memory-bound operations: add / mul / sub, copy, rmsnorm, silu
// and the host transfers.  Everything else keeps the common default
// (UnsupportedOperation, OID -2).
//
// This translation unit is plain C++20: it includes no HIP header and reaches
// the GPU only through the C ABI of libiomx (include/iomx.h).
//
// Design (not a port of src/rocm or src/shared/gpu_queue*):
//   * One device arena (a single iomx_malloc at setup, none afterwards), carved
//     by the reference's ListAllocator at 256-byte alignment.  Kernel
//     descriptors travel as kernel arguments, so there is no metadata arena and
//     no per-operation upload.
//   * A queue is one non-blocking stream, C completion events created eagerly,
//     and one completion thread.  The admission dispatch itself launches the
//     kernel and records an event (on whichever thread the common FIFO pump runs:
//     the submitting thread or the completion thread); the completion thread
//     waits for events in submission order, releases the registry entries and
//     completes the sequence.  The common layer already bounds executing work to
//     C, so an event is always free when a dispatch runs.
//   * Host transfers are synchronous, serialised per device, and stage through
//     the caller's raw workspace: host -> workspace, then the scatter kernel (or
//     the gather kernel, then workspace -> host).
#include <array>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <deque>
#include <exception>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <span>
#include <stdexcept>
#include <string>
#include <thread>
#include <type_traits>
#include <vector>

#include "iom/alloc.hpp"
#include "iom/detail/gpu_arena_config.hpp"
#include "iom/detail/outstanding_work_registry.hpp"
#include "iom/device.hpp"
#include "iom/gpu_algorithm.hpp"
#include "iom/iom.hpp"
#include "iom/rocm/device.hpp"
#include "iom/tensor.hpp"
#include "src/iom_internal.hpp"  // iom::detail::UnsupportedOperation, leaf_bits

#include "iomx.h"
#include "mi355x_testing.hpp"

namespace iom {

namespace rocm_detail {
namespace {
std::atomic<SubmissionFault> g_armed_fault{SubmissionFault::none};
}
void inject_submission_fault_for_testing(SubmissionFault fault) noexcept {
    g_armed_fault.store(fault, std::memory_order_release);
}
bool consume_submission_fault(SubmissionFault fault) noexcept {
    if (g_armed_fault.load(std::memory_order_relaxed) != fault) return false;
    SubmissionFault expected = fault;
    return g_armed_fault.compare_exchange_strong(expected, SubmissionFault::none,
                                                 std::memory_order_acq_rel);
}
std::atomic<std::size_t> event_create_count_for_testing{0};
std::atomic<std::size_t> event_destroy_count_for_testing{0};
std::atomic<std::size_t> stream_create_count_for_testing{0};
std::atomic<std::size_t> stream_destroy_count_for_testing{0};
std::atomic<std::size_t> device_allocation_count_for_testing{0};
std::atomic<std::size_t> device_free_count_for_testing{0};
std::atomic<std::size_t> linear_native_bf16_launch_count_for_testing{0};
std::atomic<std::size_t> linear_scalar_launch_count_for_testing{0};
std::atomic<std::size_t> silu_launch_count_for_testing{0};
}  // namespace rocm_detail

namespace {

using rocm_detail::SubmissionFault;
using rocm_detail::consume_submission_fault;

constexpr std::size_t kArenaAlignment = 256;
// What an injected native failure reports: hipErrorLaunchFailure's code, never raised by a kernel here.
constexpr int kInjectedDeviceError = 719;

// Counted wrappers of the native resource calls (the counters are the test seams' evidence
// that a rejected queue creates nothing and that a retained lease destroys nothing).
int counted_event_create(iomx_event_t* event) {
    if (consume_submission_fault(SubmissionFault::queue_event_create)) return kInjectedDeviceError;
    const int status = iomx_event_create(event, 0);
    if (status == IOMX_OK) rocm_detail::event_create_count_for_testing.fetch_add(1);
    return status;
}
void counted_event_destroy(iomx_event_t event) noexcept {
    (void)iomx_event_destroy(event);
    rocm_detail::event_destroy_count_for_testing.fetch_add(1);
}
int counted_stream_create(iomx_stream_t* stream) {
    if (consume_submission_fault(SubmissionFault::queue_stream_create)) return kInjectedDeviceError;
    const int status = iomx_stream_create(stream);
    if (status == IOMX_OK) rocm_detail::stream_create_count_for_testing.fetch_add(1);
    return status;
}
void counted_stream_destroy(iomx_stream_t stream) noexcept {
    if (stream == nullptr) return;
    (void)iomx_stream_destroy(stream);
    rocm_detail::stream_destroy_count_for_testing.fetch_add(1);
}

// A callable with in-place storage: the per-operation completion actions capture a few
// registry ids and references, and a std::function would put them on the heap once per
// operation.  Captures must be trivially copyable, so a move is a byte copy.
template <typename Signature, std::size_t Bytes>
class InlineFunction;
template <typename R, typename... A, std::size_t Bytes>
class InlineFunction<R(A...), Bytes> {
public:
    InlineFunction() = default;
    template <typename F, typename = std::enable_if_t<!std::is_same_v<std::decay_t<F>, InlineFunction>>>
    InlineFunction(F f) {  // NOLINT: implicit on purpose, like std::function
        static_assert(sizeof(F) <= Bytes, "capture does not fit the in-place storage");
        static_assert(std::is_trivially_copyable_v<F> && std::is_trivially_destructible_v<F>,
                      "captures must be plain data");
        new (storage_) F(f);
        invoke_ = [](void* self, A... args) -> R { return (*static_cast<F*>(self))(args...); };
    }
    explicit operator bool() const noexcept { return invoke_ != nullptr; }
    R operator()(A... args) { return invoke_(storage_, args...); }
private:
    alignas(std::max_align_t) unsigned char storage_[Bytes] = {};
    R (*invoke_)(void*, A...) = nullptr;
};

[[noreturn]] void throw_status(int status, const char* what) {
    std::string message(what);
    message += ": ";
    message += iomx_error_string(status);
    if (status == IOMX_ERR_INVALID) throw std::invalid_argument(message);
    if (status == IOMX_ERR_OVERFLOW) throw std::overflow_error(message);
    if (status == IOMX_ERR_UNSUPPORTED) throw detail::UnsupportedOperation();
    throw std::runtime_error(message);
}

void check(int status, const char* what) {
    if (status != IOMX_OK) throw_status(status, what);
}

// Leaf codes of the C ABI are the numeric values of iom::DataType.  Every leaf
// is stored, copied and transferred; the 21 numeric leaves take the binary
// operations (src/device_ops_binary.cpp:26-46); the 9 floating leaves take
// rmsnorm and silu (F8_E8M0 is a scale encoding, not a number).
int transfer_code(DataType type) {
    const int code = static_cast<int>(type);
    return (code >= 0 && code <= static_cast<int>(DataType::F64)) ? code : -1;
}

int binary_code(DataType type) {
    if (type == DataType::BOOL || type == DataType::F8_E8M0) return -1;
    return transfer_code(type);
}

int float_code(DataType type) {
    switch (type) {
        case DataType::F4_E2M1: case DataType::F6_E2M3: case DataType::F6_E3M2:
        case DataType::F8_E4M3FN: case DataType::F8_E5M2: case DataType::F16:
        case DataType::BF16: case DataType::F32: case DataType::F64:
            return static_cast<int>(type);
        default:
            return -1;
    }
}

// The 23 leaves of every standard tiled backend, in the order the reference
// publishes them (src/shared/standard_tiled_copy.hpp:17-31).
constexpr std::array<DataType, 23> kStoredLeaves = {
        DataType::BOOL,
        DataType::I2, DataType::U2, DataType::I4, DataType::U4, DataType::I8, DataType::U8,
        DataType::I16, DataType::U16, DataType::I32, DataType::U32, DataType::I64, DataType::U64,
        DataType::F4_E2M1, DataType::F6_E2M3, DataType::F6_E3M2,
        DataType::F8_E4M3FN, DataType::F8_E5M2, DataType::F8_E8M0,
        DataType::F16, DataType::BF16, DataType::F32, DataType::F64};

iomx_view make_view(void* base, std::span<const std::size_t> dims, std::size_t plane_offset,
                    std::span<const std::size_t> plane_strides) {
    iomx_view v{};
    v.base = base;
    v.rank = static_cast<std::uint32_t>(dims.size());
    for (std::size_t i = 0; i < dims.size(); ++i) v.dims[i] = dims[i];
    v.plane_offset = plane_offset;
    for (std::size_t i = 0; i + 2 < dims.size() && i < plane_strides.size(); ++i)
        v.plane_strides[i] = plane_strides[i];
    return v;
}

iomx_view make_view(const TensorView& view) {
    return make_view(const_cast<void*>(view.native_handle()), view.spec().shape.dimensions(),
                     view.plane_offset(), view.plane_strides());
}

class Mi355xDevice;

// ---------------------------------------------------------------------------
// Device
// ---------------------------------------------------------------------------

class Mi355xDevice final : public Device {
public:
    Mi355xDevice(std::uint32_t ordinal, std::size_t arena_bytes, QueueConfig queue_config)
            : Device(queue_config), ordinal_(ordinal), arena_bytes_(arena_bytes) {
        int count = 0;
        if (iomx_device_count(&count) != IOMX_OK || ordinal >= static_cast<std::uint32_t>(count))
            throw std::invalid_argument("MI355X device ordinal does not exist");
        check(iomx_set_device(static_cast<int>(ordinal_)), "set device");
        if (iomx_malloc(&arena_, arena_bytes_) != IOMX_OK || arena_ == nullptr)
            throw std::bad_alloc();
        rocm_detail::device_allocation_count_for_testing.fetch_add(1);
        try {
            allocator_ = std::make_unique<ListAllocator>(arena_, arena_bytes_, kArenaAlignment);
            check(iomx_stream_create(&transfer_stream_), "transfer stream");
        } catch (...) {
            (void)iomx_free(arena_);
            rocm_detail::device_free_count_for_testing.fetch_add(1);
            throw;
        }
    }

    ~Mi355xDevice() override {
        (void)iomx_set_device(static_cast<int>(ordinal_));
        if (transfer_stream_ != nullptr) {
            (void)iomx_stream_synchronize(transfer_stream_);
            (void)iomx_stream_destroy(transfer_stream_);
        }
        // Leases that a failed final synchronisation left here: the device-wide
        // synchronisation below is their covering proof; either way they end with the device.
        (void)iomx_device_synchronize();
        discard_retained_leases();
        // Quarantined storage is returned to the allocator's host-side books when
        // the registry state is destroyed (after this body); the device range
        // itself can go now.
        (void)iomx_free(arena_);
        rocm_detail::device_free_count_for_testing.fetch_add(1);
    }

    [[nodiscard]] BackendKind backend_kind() const noexcept override { return BackendKind::ROCM; }
    [[nodiscard]] std::uint32_t backend_device() const noexcept override { return ordinal_; }
    [[nodiscard]] std::span<const DataType> supported_data_types() const noexcept override {
        return kStoredLeaves;
    }

    [[nodiscard]] std::unique_ptr<Tensor> create_tensor(const TensorSpec& spec) override;
    [[nodiscard]] std::unique_ptr<RawWorkspace> create_workspace(std::size_t bytes) override;
    [[nodiscard]] std::unique_ptr<DeviceOps> create_ops() override;

    [[nodiscard]] detail::RegistryState& registry_state() noexcept { return registry_state_; }
    [[nodiscard]] int ordinal() const noexcept { return static_cast<int>(ordinal_); }

    // Arena suballocation; exhaustion (including fragmentation) is std::bad_alloc.
    [[nodiscard]] void* allocate(std::size_t bytes) {
        std::lock_guard<std::mutex> lock(arena_mutex_);
        void* address = allocator_->alloc(bytes);
        if (address == nullptr) throw std::bad_alloc();
        return address;
    }
    void release(void* address) noexcept {
        if (address == nullptr) return;
        std::lock_guard<std::mutex> lock(arena_mutex_);
        try { allocator_->free(address); } catch (...) {}
    }
    [[nodiscard]] Allocator& data_allocator() noexcept { return *guarded_allocator_; }

    // A workspace owner goes away (src/rocm/device.cpp:243-264).  A range that an accepted
    // operation still leases -- the caller dropped the workspace before it waited -- must not
    // return to the allocator while the kernel may use it: it is parked in the quarantine,
    // which gives it back at the device's end.
    void release_workspace(const RawWorkspace* owner, void* address, std::size_t bytes) noexcept {
        if (address == nullptr) return;
        bool retained = false;
        {
            std::lock_guard<std::mutex> lock(registry_state_.allocation_mutex);
            retained = detail::workspace_range_retained(registry_state_.workspace_leases, owner,
                                                        address, bytes);
        }
        if (retained) {
            try {
                registry_state_.quarantine.emplace<detail::AllocatorCleanupAction>(
                        *guarded_allocator_, address, bytes);
            } catch (...) {
                // the range simply stays unavailable
            }
            return;
        }
        release(address);
    }

    // src/rocm/device_tensor.cpp:22-41: storage handed to a tensor is device memory of this
    // ordinal inside this device's arena.
    void validate_storage(void* address) const {
        int owner = -1;
        const int status = iomx_pointer_device(address, &owner);
        const std::uintptr_t raw = reinterpret_cast<std::uintptr_t>(address);
        const std::uintptr_t base = reinterpret_cast<std::uintptr_t>(arena_);
        if (status != IOMX_OK || owner != ordinal() || raw < base || raw - base >= arena_bytes_)
            throw std::runtime_error("MI355X tensor storage is incompatible with the owning device");
    }

    // ---- queue leases whose completion could not be proved ---------------------------
    // (src/shared/gpu_queue_lifecycle.inl:94-180)  A queue whose final stream synchronisation
    // fails leaves its stream, completion events, status cells and its place among the four
    // queues here.  Nothing of it is destroyed or reused until a later synchronisation of that
    // same stream succeeds (reclaim) or the device ends.
    struct QueueLease {
        iomx_stream_t stream = nullptr;
        std::vector<iomx_event_t> events;
        std::uint32_t* status_cells = nullptr;
    };
    static void destroy_lease(QueueLease& lease) noexcept {
        for (iomx_event_t event : lease.events) counted_event_destroy(event);
        lease.events.clear();
        counted_stream_destroy(lease.stream);
        lease.stream = nullptr;
        if (lease.status_cells != nullptr) (void)iomx_host_free(lease.status_cells);
        lease.status_cells = nullptr;
    }
    void retain_unknown_lease(QueueLease lease) noexcept {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        try {
            retained_leases_.push_back(std::move(lease));
        } catch (...) {
            // no room to remember it: the native objects stay alive, unreferenced
        }
    }
    void reclaim_retained_leases() noexcept {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        (void)iomx_set_device(ordinal());
        for (std::size_t i = 0; i < retained_leases_.size();) {
            const bool proved = !consume_submission_fault(SubmissionFault::stream_synchronize)
                    && iomx_stream_synchronize(retained_leases_[i].stream) == IOMX_OK;
            if (!proved) { ++i; continue; }
            destroy_lease(retained_leases_[i]);
            retained_leases_.erase(retained_leases_.begin() + static_cast<std::ptrdiff_t>(i));
        }
    }
    void discard_retained_leases() noexcept {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        for (QueueLease& lease : retained_leases_) destroy_lease(lease);
        retained_leases_.clear();
    }
    [[nodiscard]] std::size_t retained_lease_count() noexcept {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        return retained_leases_.size();
    }
    // A retained lease keeps its place among the device's four queues: together with the
    // live queues (counted by the common layer) it may not exceed four.
    void admit_queue() {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        if (live_queues_ + retained_leases_.size() >= 4) throw std::bad_alloc();
        ++live_queues_;
    }
    void retire_queue() noexcept {
        std::lock_guard<std::mutex> lock(retained_mutex_);
        if (live_queues_ != 0) --live_queues_;
    }

    // Host transfers: one at a time per device, never waiting on any queue.
    void transfer(const TensorView& view, RawWorkspaceView workspace,
                  std::span<const std::byte> source, std::span<std::byte> destination,
                  bool from_host) {
        const WorkspaceRequirements need = view.copy_from_host_workspace_requirements();
        const std::array<TensorView, 1> operands{view};
        const RawWorkspaceView checked = detail::WorkspaceValidation::validated(
                *this, workspace, need.bytes, need.alignment, operands);
        void* staging = detail::WorkspaceValidation::address(checked);
        const int code = transfer_code(view.spec().data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        const std::size_t nbytes = view.spec().logical_nbytes();
        const iomx_view v = make_view(view);
        std::lock_guard<std::mutex> lock(transfer_mutex_);
        if (transfer_poisoned_) throw std::bad_alloc();
        try {
            check(iomx_set_device(ordinal()), "set device");
            if (from_host) {
                check(iomx_memcpy_h2d(staging, source.data(), nbytes), "host to staging");
                check(iomx_launch_scatter(code, &v, staging, transfer_stream_), "scatter");
                check(iomx_stream_synchronize(transfer_stream_), "scatter completion");
            } else {
                check(iomx_launch_gather(code, &v, staging, transfer_stream_), "gather");
                check(iomx_stream_synchronize(transfer_stream_), "gather completion");
                check(iomx_memcpy_d2h(destination.data(), staging, nbytes), "staging to host");
            }
        } catch (...) {
            transfer_poisoned_ = true;  // a failed transfer leaves the stream's state unknown
            throw;
        }
    }

    void zero_fill(void* address, std::size_t bytes) {
        std::lock_guard<std::mutex> lock(transfer_mutex_);
        check(iomx_set_device(ordinal()), "set device");
        check(iomx_fill_async(address, 0, bytes, transfer_stream_), "zero fill");
        check(iomx_stream_synchronize(transfer_stream_), "zero fill completion");
    }

private:
    // Allocator facade whose free() takes the arena lock: quarantined storage is
    // released through it from whatever thread drains the quarantine.
    class GuardedAllocator final : public Allocator {
    public:
        explicit GuardedAllocator(Mi355xDevice& device) : device_(device) {}
        void* alloc(std::size_t bytes) override { return device_.allocate(bytes); }
        void free(void* address) override { device_.release(address); }
        void reset() override {}
    private:
        Mi355xDevice& device_;
    };

    std::uint32_t ordinal_;
    std::size_t arena_bytes_;
    void* arena_ = nullptr;
    std::mutex arena_mutex_;
    std::unique_ptr<ListAllocator> allocator_;
    std::unique_ptr<GuardedAllocator> guarded_allocator_ = std::make_unique<GuardedAllocator>(*this);
    iomx_stream_t transfer_stream_ = nullptr;
    std::mutex transfer_mutex_;
    bool transfer_poisoned_ = false;
    std::mutex retained_mutex_;
    std::vector<QueueLease> retained_leases_;
    std::size_t live_queues_ = 0;
    // Destroyed first (declared last): draining its quarantine uses the allocator.
    detail::RegistryState registry_state_;
};

// ---------------------------------------------------------------------------
// Tensor and workspace owners
// ---------------------------------------------------------------------------

class Mi355xTensor final : public Tensor {
public:
    Mi355xTensor(const TensorSpec& spec, Mi355xDevice& device)
            : Tensor(spec, device), device_(device) {
        if (transfer_code(spec.data_type) < 0) throw detail::UnsupportedOperation();
        bytes_ = view().spec().tiled_storage_nbytes();
        address_ = device_.allocate(bytes_);
        try {
            device_.validate_storage(address_);
            device_.zero_fill(address_, bytes_);
        } catch (...) {
            device_.release(address_);
            throw;
        }
    }

    ~Mi355xTensor() noexcept override {
        if (address_ == nullptr) return;
        void* address = address_;
        // Storage with unproven outstanding work is parked in the quarantine and
        // returned to the arena only when the device goes away
        // (include/iom/detail/outstanding_work_registry_core.hpp:235-275).
        detail::release_or_quarantine(
                device_.registry_state().registry, address,
                [this, address] {
                    try {
                        device_.registry_state().quarantine
                                .emplace<detail::AllocatorCleanupAction>(
                                        device_.data_allocator(), address, bytes_);
                    } catch (...) {
                    }
                    address_ = nullptr;
                },
                [this, address] {
                    device_.release(address);
                    address_ = nullptr;
                });
    }

private:
    [[nodiscard]] void* storage_handle() noexcept override { return address_; }
    [[nodiscard]] WorkspaceRequirements host_transfer_workspace_requirements(
            std::size_t checked_logical_nbytes) const override {
        return {gpu_algorithm::compute_staging_size(checked_logical_nbytes), 32};
    }
    void region_from_host(const TensorView& destination, std::span<const std::byte> source,
                          RawWorkspaceView workspace) override {
        device_.transfer(destination, workspace, source, {}, true);
    }
    void region_to_host(const TensorView& source, std::span<std::byte> destination,
                        RawWorkspaceView workspace) const override {
        device_.transfer(source, workspace, {}, destination, false);
    }

    Mi355xDevice& device_;
    void* address_ = nullptr;
    std::size_t bytes_ = 0;
};

class Mi355xWorkspace final : public RawWorkspace {
public:
    Mi355xWorkspace(Mi355xDevice& device, std::size_t bytes)
            : RawWorkspace(device, bytes), device_(device) {
        if (bytes != 0) address_ = device_.allocate(bytes);
    }
    ~Mi355xWorkspace() noexcept override { device_.release_workspace(this, address_, byte_size()); }

private:
    [[nodiscard]] void* workspace_address() const noexcept override { return address_; }
    Mi355xDevice& device_;
    void* address_ = nullptr;
};

// ---------------------------------------------------------------------------
// Queue
// ---------------------------------------------------------------------------

class Mi355xQueue final : public DeviceOps {
public:
    explicit Mi355xQueue(Mi355xDevice& device)
            : DeviceOps(device), device_(device),
              registry_queue_id_(detail::allocate_queue_id(device.registry_state())) {
        const std::size_t capacity = device.queue_config().max_in_flight_per_queue;
        // a lease retained by an earlier queue keeps its place: refused before any native resource
        device_.admit_queue();
        try {
            check(iomx_set_device(device_.ordinal()), "set device");
            events_.reserve(capacity);
            free_events_.reserve(capacity);
            for (std::size_t i = 0; i < capacity; ++i) {
                iomx_event_t event = nullptr;
                check(counted_event_create(&event), "completion event");
                events_.push_back(event);
                free_events_.push_back(event);
            }
            // one page-locked status word per completion event (the embedding lookup
            // reports an invalid id through it,
            // docs/BACKEND_CONTRACT/embedding-lookup.md:178-203)
            // and one completion word per event behind them: an operation submitted to an idle
            // queue signals through its word, which the completion thread sees earlier than
            // the event (see start())
            void* cells = nullptr;
            check(iomx_host_alloc(&cells, 2 * capacity * sizeof(std::uint32_t)), "status cells");
            status_cells_ = static_cast<std::uint32_t*>(cells);
            std::memset(status_cells_, 0, 2 * capacity * sizeof(std::uint32_t));
            void* device_side = nullptr;
            check(iomx_host_device_address(status_cells_, &device_side), "status cells");
            cells_on_device_ = static_cast<std::uint32_t*>(device_side);
            check(counted_stream_create(&stream_), "queue stream");
            completer_ = std::thread([this] { run_completer(); });
        } catch (...) {
            destroy_native();
            device_.retire_queue();
            throw;
        }
    }

    ~Mi355xQueue() override {
        // Owner fences of this queue's outstanding work are invalidated before anything drains
        // (src/shared/gpu_queue_lifecycle.inl:96-101): an operand of accepted work that nobody
        // waited for, destroyed after its queue, is then quarantined until the device ends
        // instead of depending on how far the drain below happened to get.
        device_.registry_state().registry.invalidate_entries_for_queue(registry_queue_id_);
        // Stop accepting, fail what never started, then let the completion thread
        // finish everything that was launched before the native objects go away.
        close_and_drain();
        {
            std::unique_lock<std::mutex> lock(mutex_);
            shutdown_ = true;
        }
        cv_.notify_all();
        if (completer_.joinable()) completer_.join();
        close_and_drain();
        (void)iomx_set_device(device_.ordinal());
        // The final proof that nothing of this queue still runs.  Without it nothing native is
        // destroyed or reused: the whole lease moves to the device, keeps its place among the
        // four queues, and ends at a later proof on the same stream or with the device.
        const bool proved = stream_ == nullptr
                || (!consume_submission_fault(SubmissionFault::stream_synchronize)
                    && iomx_stream_synchronize(stream_) == IOMX_OK);
        release_unobserved_leases(proved);
        if (proved) {
            destroy_native();
        } else {
            Mi355xDevice::QueueLease lease;
            lease.stream = stream_;
            lease.events = std::move(events_);
            lease.status_cells = status_cells_;
            stream_ = nullptr;
            events_.clear();
            free_events_.clear();
            status_cells_ = nullptr;
            device_.retain_unknown_lease(std::move(lease));
        }
        device_.retire_queue();
        device_.registry_state().registry.invalidate_entries_for_queue(registry_queue_id_);
    }

    void snapshot(rocm_detail::QueueResourceSnapshot& out) {
        std::lock_guard<std::mutex> lock(mutex_);
        out.events_total = events_.size();
        out.events_in_use = events_.size() - free_events_.size();
        out.operations_in_flight = in_flight_.size() + (completing_ ? 1 : 0);
    }

    [[nodiscard]] std::string_view backend_label() const noexcept override { return "MI355X"; }

private:
    // What completion does with the operation's registry entries and workspace lease.
    // failed: the operation's terminal state is a failure.  proved: the device has provably
    // finished with the operands (the completion event or word was seen, or the stream was
    // synchronised after a failed submission); without proof owners and workspace ranges are
    // quarantined instead of released (src/shared/gpu_queue_operations.inl:1031-1046).
    using Finish = InlineFunction<void(bool failed, bool proved), 160>;

    // After native completion: turns a data error the kernel reported into the
    // operation's retained failure (null = none).
    using Verify = std::exception_ptr (*)(std::uint32_t status);

    struct InFlight {
        std::uint64_t sequence = 0;
        iomx_event_t event = nullptr;
        std::uint32_t* status = nullptr;
        std::uint32_t* word = nullptr;      // completion word, or null: completion by the event
        std::uint32_t ticket = 0;
        std::exception_ptr failure;
        Finish finish;
        Verify verify = nullptr;
        bool deny_proof = false;            // test seam: the proving synchronisation fails too
    };

    static detail::FenceResult fence_pending(const detail::Fence&) noexcept {
        return detail::FenceResult::pending();
    }
    [[nodiscard]] static detail::Fence pending_fence() noexcept {
        detail::Fence fence;
        fence.invoke = &fence_pending;
        return fence;
    }

    void destroy_native() noexcept {
        for (iomx_event_t event : events_) counted_event_destroy(event);
        events_.clear();
        free_events_.clear();
        counted_stream_destroy(stream_);
        stream_ = nullptr;
        if (status_cells_ != nullptr) (void)iomx_host_free(status_cells_);
        status_cells_ = nullptr;
    }

    [[nodiscard]] std::uint32_t* status_cell(iomx_event_t event) noexcept {
        for (std::size_t i = 0; i < events_.size(); ++i)
            if (events_[i] == event) return status_cells_ + i;
        return nullptr;
    }
    [[nodiscard]] std::uint32_t* completion_word(iomx_event_t event) noexcept {
        std::uint32_t* cell = status_cell(event);
        return cell == nullptr ? nullptr : cell + events_.size();
    }

    // Runs inside the common admission dispatch: launch on the queue stream,
    // record the completion event, hand the rest to the completion thread.
    // Throws only before anything was launched.
    template <typename Launch>
    void start(std::uint64_t sequence, Launch&& launch, Finish finish, Verify verify = nullptr) {
        // a completion resource that cannot be had is a failure before acceptance: the common
        // layer rolls the request back and reports a device error (OID -5)
        if (consume_submission_fault(SubmissionFault::event_create))
            throw std::runtime_error("MI355X completion resource is unavailable (injected)");
        iomx_event_t event = nullptr;
        // An operation that finds the queue idle is most likely one its caller is about to wait
        // for (the session submits, waits, submits: src/session.cpp:2000-2045): it signals through
        // a completion word, which costs the submitting thread 1.7 us more than recording the
        // event and reaches the completion thread 4 us earlier.  Behind other operations the
        // event is recorded: there the submitting thread is the one that must not be held up.
        bool idle = false;
        std::uint32_t ticket = 0;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (shutdown_) throw std::logic_error("MI355X queue is shut down");
            if (free_events_.empty()) throw detail::AdmissionResourceUnavailable();
            event = free_events_.back();
            free_events_.pop_back();
            idle = in_flight_.empty() && !completing_;
            if (idle && ++ticket_ == 0) ++ticket_;
            ticket = ticket_;
        }
        InFlight item;
        item.sequence = sequence;
        item.event = event;
        if (idle) {
            item.word = completion_word(event);
            item.ticket = ticket;
        }
        item.finish = finish;
        item.verify = verify;
        item.status = status_cell(event);
        int status = iomx_set_device(device_.ordinal());
        if (status == IOMX_OK) {
            if (consume_submission_fault(SubmissionFault::kernel_launch))
                status = kInjectedDeviceError;      // the launch is not made
            else if constexpr (std::is_invocable_v<Launch&, iomx_stream_t, std::uint32_t*>)
                status = launch(stream_, item.status);
            else
                status = launch(stream_);
        }
        if (status == IOMX_OK) {
            if (consume_submission_fault(SubmissionFault::event_record)) status = kInjectedDeviceError;
            else if (consume_submission_fault(SubmissionFault::event_record_unproved)) {
                status = kInjectedDeviceError;
                item.deny_proof = true;
            } else if (item.word != nullptr)
                status = iomx_stream_write_word(stream_, cells_on_device_ + (item.word - status_cells_), item.ticket);
            else status = iomx_event_record(event, stream_);
        }
        if (status != IOMX_OK) {
            try { throw_status(status, "MI355X kernel submission"); }
            catch (...) { item.failure = std::current_exception(); }
        }
        bool wake = false;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            in_flight_.push_back(std::move(item));
            pending_.store(in_flight_.size(), std::memory_order_release);
            wake = completer_sleeping_;
        }
        if (wake) cv_.notify_one();
    }

    static void relax() noexcept {
#if defined(__x86_64__) || defined(__i386__)
        __builtin_ia32_pause();
#endif
    }

    // The next launched operation, in submission order.  The completion thread polls for a
    // short while before it sleeps: a session that submits one operation, waits and submits the
    // next (src/session.cpp:2000-2045) then never pays a thread wake-up per operation.
    bool next_in_flight(InFlight& item) {
        const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(150);
        for (unsigned spins = 0;; ++spins) {
            if (pending_.load(std::memory_order_acquire) != 0) {
                std::lock_guard<std::mutex> lock(mutex_);
                if (!in_flight_.empty()) {
                    item = std::move(in_flight_.front());
                    in_flight_.pop_front();
                    pending_.store(in_flight_.size(), std::memory_order_release);
                    completing_ = true;
                    return true;
                }
            }
            if ((spins & 63u) == 63u && std::chrono::steady_clock::now() > give_up) break;
            relax();
        }
        std::unique_lock<std::mutex> lock(mutex_);
        completer_sleeping_ = true;
        cv_.wait(lock, [this] { return shutdown_ || !in_flight_.empty(); });
        completer_sleeping_ = false;
        if (in_flight_.empty()) return false;
        item = std::move(in_flight_.front());
        in_flight_.pop_front();
        pending_.store(in_flight_.size(), std::memory_order_release);
        completing_ = true;
        return true;
    }

    // Completion of one event: polled while the kernel is short, then a blocking wait.
    [[nodiscard]] static int await_event(iomx_event_t event) noexcept {
        const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(300);
        for (unsigned spins = 0;; ++spins) {
            int done = 0;
            const int status = iomx_event_query(event, &done);
            if (status != IOMX_OK) return status;
            if (done) return IOMX_OK;
            if ((spins & 15u) == 15u && std::chrono::steady_clock::now() > give_up) break;
            relax();
        }
        return iomx_event_synchronize(event);
    }

    // Completion through the word: polled like the event; a word that has not arrived within
    // the polling time is waited for on the stream, which also reports what went wrong.
    [[nodiscard]] int await_word(const std::uint32_t* word, std::uint32_t ticket) noexcept {
        const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(300);
        for (unsigned spins = 0;; ++spins) {
            if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == ticket) return IOMX_OK;
            if ((spins & 63u) == 63u && std::chrono::steady_clock::now() > give_up) break;
            relax();
        }
        return iomx_stream_synchronize(stream_);
    }

    void run_completer() noexcept {
        (void)iomx_set_device(device_.ordinal());
        for (;;) {
            InFlight item;
            if (!next_in_flight(item)) return;
            bool proved = true;
            if (!item.failure) {
                const int status = item.word != nullptr ? await_word(item.word, item.ticket)
                                                        : await_event(item.event);
                if (status != IOMX_OK) {
                    try { throw_status(status, "MI355X kernel completion"); }
                    catch (...) { item.failure = std::current_exception(); }
                    // the wait itself failed: only a synchronisation of the stream can still
                    // show that the kernel is done with its operands
                    proved = iomx_stream_synchronize(stream_) == IOMX_OK;
                } else if (item.verify != nullptr) {
                    // a native failure takes precedence over the status word
                    item.failure = item.verify(*item.status);
                }
            } else {
                // The submission failed after its launch (or with earlier work still on the
                // stream): nothing signals its end, so the stream is synchronised -- which also
                // keeps completion in order -- and only a successful synchronisation proves that
                // the operands are free.
                proved = !item.deny_proof && iomx_stream_synchronize(stream_) == IOMX_OK;
            }
            {
                std::lock_guard<std::mutex> lock(mutex_);
                free_events_.push_back(item.event);
                completing_ = false;
            }
            try { if (item.finish) item.finish(static_cast<bool>(item.failure), proved); } catch (...) {}
            try { complete(item.sequence, std::move(item.failure)); } catch (...) {}
        }
    }

    // Workspace leases of finished attention requests that no caller has observed yet.
    [[nodiscard]] bool keep_until_observed(std::uint64_t sequence, const detail::WorkspaceLease& lease) noexcept {
        try {
            std::lock_guard<std::mutex> lock(observed_mutex_);
            return unobserved_leases_.emplace(sequence, lease).second;
        } catch (...) {
            return false;
        }
    }

    // wait() has seen the token's terminal state: its workspace range may be leased again
    // (src/shared/gpu_queue_operations.inl:1188-1205).  Repeated waits find nothing.
    void fence_through_sequence(std::uint64_t sequence) noexcept override {
        detail::WorkspaceLease lease{};
        {
            std::lock_guard<std::mutex> lock(observed_mutex_);
            const auto found = unobserved_leases_.find(sequence);
            if (found == unobserved_leases_.end()) return;
            lease = found->second;
            unobserved_leases_.erase(found);
        }
        detail::complete_workspace_lease(device_.registry_state(), lease, true);
    }

    // Queue teardown: whatever no caller observed (src/shared/gpu_queue_operations.inl:1207-1226).
    void release_unobserved_leases(bool covering_proof) noexcept {
        std::map<std::uint64_t, detail::WorkspaceLease> leases;
        try {
            std::lock_guard<std::mutex> lock(observed_mutex_);
            leases.swap(unobserved_leases_);
        } catch (...) {
            return;   // the ranges stay reserved, never reused unsafely
        }
        for (const auto& entry : leases)
            detail::complete_workspace_lease(device_.registry_state(), entry.second, covering_proof);
    }

    // ---- hooks ----------------------------------------------------------------

    oid copy_impl(const TensorView& source, TensorView& destination) override {
        const int code = transfer_code(source.spec().data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_copy(
                source, destination, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const CopyRequest& captured,
                             detail::EntryRegistration entries) {
                    auto& registry = device_.registry_state().registry;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  if (captured.no_op) return static_cast<int>(IOMX_OK);
                                  const iomx_view src = make_view(
                                          captured.source.native_handle,
                                          captured.source.spec.shape.dimensions(),
                                          captured.source.plane_offset, captured.source.plane_strides);
                                  const iomx_view dst = make_view(
                                          captured.destination.native_handle,
                                          captured.destination.spec.shape.dimensions(),
                                          captured.destination.plane_offset,
                                          captured.destination.plane_strides);
                                  return iomx_launch_copy(code, &src, &dst, stream);
                              },
                              [&registry, entries](bool failed, bool proved) {
                                  const detail::SequenceOutcome outcome{
                                          entries.source, entries.destination, nullptr, true};
                                  (void)detail::release_or_invalidate_entries(
                                          registry, outcome, failed, proved);
                              });
                    } catch (...) {
                        registry.remove_entry_if_present(
                                entries.source, captured.source.native_handle);
                        registry.remove_entry_if_present(
                                entries.destination, captured.destination.native_handle);
                        throw;
                    }
                });
    }

    oid binary_impl(const BinaryRequest& request) override {
        const int code = binary_code(request.out.spec.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        int op = IOMX_OP_ADD;
        if (request.operation == BinaryOperation::Mul) op = IOMX_OP_MUL;
        if (request.operation == BinaryOperation::Sub) op = IOMX_OP_SUB;
        if (request.operation == BinaryOperation::Div) op = IOMX_OP_DIV;
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_binary(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code, op](std::uint64_t sequence, const BinaryRequest& captured,
                                 detail::BinaryEntryRegistration entries) {
                    auto& state = device_.registry_state();
                    const detail::WorkspaceLease lease = captured.workspace_lease;
                    try {
                        start(sequence,
                              [&captured, code, op](iomx_stream_t stream) {
                                  const auto view_of = [](const BinaryViewSnapshot& s) {
                                      return make_view(s.native_handle, s.spec.shape.dimensions(),
                                                       s.plane_offset, s.plane_strides);
                                  };
                                  const iomx_view lhs = view_of(captured.lhs);
                                  const iomx_view rhs = view_of(captured.rhs);
                                  const iomx_view out = view_of(captured.out);
                                  return iomx_launch_binary(op, code, &lhs, &rhs, &out, stream);
                              },
                              [&state, entries, lease](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          state.registry, entries, failed, proved);
                                  detail::complete_workspace_lease(state, lease, proved);
                              });
                    } catch (...) {
                        state.registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        detail::complete_workspace_lease(state, lease, true);
                        throw;
                    }
                });
    }

    [[nodiscard]] bool rmsnorm_supported(DataType data_type) const override {
        return float_code(data_type) >= 0;
    }

    oid rmsnorm_impl(const RmsnormRequest& request) override {
        const int code = float_code(request.x.spec.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_rmsnorm(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const RmsnormRequest& captured,
                             detail::BinaryEntryRegistration entries) {
                    auto& registry = device_.registry_state().registry;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  const auto view_of = [](const CopyViewSnapshot& s) {
                                      return make_view(s.native_handle, s.spec.shape.dimensions(),
                                                       s.plane_offset, s.plane_strides);
                                  };
                                  const iomx_view x = view_of(captured.x);
                                  const iomx_view scale = view_of(captured.scale);
                                  const iomx_view out = view_of(captured.out);
                                  return iomx_launch_rmsnorm(code, &x, &scale, &out,
                                                             captured.epsilon, stream);
                              },
                              [&registry, entries](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          registry, entries, failed, proved);
                              });
                    } catch (...) {
                        registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        throw;
                    }
                });
    }

    // ---- linear projection --------------------------------------------------------

    [[nodiscard]] WorkspaceRequirements linear_workspace_requirements_impl(
            const TensorView& x, const TensorView&, const TensorView&, std::size_t, std::size_t,
            LinearOutputLayout, std::size_t, std::size_t) override {
        if (binary_code(x.spec().data_type) < 0) throw detail::UnsupportedOperation();
        return {0, 1};
    }

    oid linear_impl(const LinearRequest& request) override {
        const int code = binary_code(request.x.spec.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        if (!request.workspace.empty())
            throw std::invalid_argument("MI355X linear projection consumes no raw workspace");
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_linear(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const LinearRequest& captured,
                             detail::BinaryEntryRegistration entries) {
                    auto& state = device_.registry_state();
                    const detail::WorkspaceLease lease = captured.workspace_lease;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  const auto view_of = [](const LinearViewSnapshot& s) {
                                      return make_view(s.native_handle, s.spec.shape.dimensions(),
                                                       s.plane_offset, s.plane_strides);
                                  };
                                  const iomx_view x = view_of(captured.x);
                                  const iomx_view w = view_of(captured.w);
                                  const iomx_view out = view_of(captured.out);
                                  const bool planar = captured.layout == LinearOutputLayout::head_planar;
                                  const int status = iomx_launch_linear(
                                          code, &x, &w, &out, captured.start_row, captured.rows,
                                          planar ? 1 : 0, captured.heads, captured.head_dim, 0, stream);
                                  iomx_launch_info info{};
                                  if (status == IOMX_OK && iomx_last_launch(&info) == IOMX_OK) {
                                      const std::string_view kernel(info.kernel);
                                      if (kernel.rfind("linear_mfma", 0) == 0)
                                          rocm_detail::linear_native_bf16_launch_count_for_testing.fetch_add(1);
                                      else
                                          rocm_detail::linear_scalar_launch_count_for_testing.fetch_add(1);
                                  }
                                  return status;
                              },
                              [&state, entries, lease](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          state.registry, entries, failed, proved);
                                  detail::complete_workspace_lease(state, lease, proved);
                              });
                    } catch (...) {
                        state.registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        detail::complete_workspace_lease(state, lease, true);
                        throw;
                    }
                });
    }

    // ---- attention ----------------------------------------------------------------

    // BF16 only (docs/BACKEND_CONTRACT/scaled-dot-product-attention.md "Current capability
    // matrix"); every other leaf is an explicit rejection after structural validation.
    [[nodiscard]] WorkspaceRequirements sdpa_workspace_requirements_impl(
            const SdpaRequest& request) override {
        if (request.q.data_type != DataType::BF16) throw detail::UnsupportedOperation();
        const iomx_view q = snapshot_view(request.q), k = snapshot_view(request.k);
        const iomx_view v = snapshot_view(request.v), out = snapshot_view(request.out);
        std::uint64_t bytes = 0, alignment = 1;
        const int status = iomx_sdpa_workspace(IOMX_DT_BF16, &q, &k, &v, &out, request.a, request.L,
                                               &bytes, &alignment);
        if (status == IOMX_ERR_UNSUPPORTED) throw detail::UnsupportedOperation();
        if (status != IOMX_OK) throw std::length_error("MI355X SDPA workspace size overflows");
        return {static_cast<std::size_t>(bytes), static_cast<std::size_t>(alignment)};
    }

    oid sdpa_impl(const SdpaRequest& request) override {
        if (request.q.data_type != DataType::BF16) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_sdpa(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this](std::uint64_t sequence, const SdpaRequest& captured,
                       detail::SdpaEntryRegistration entries) {
                    auto& state = device_.registry_state();
                    const detail::WorkspaceLease lease = captured.workspace_lease;
                    try {
                        void* scratch = captured.workspace.empty()
                                ? nullptr : detail::WorkspaceValidation::address(captured.workspace);
                        const std::uint64_t scratch_bytes = captured.workspace.byte_size();
                        start(sequence,
                              [&captured, scratch, scratch_bytes](iomx_stream_t stream) {
                                  const iomx_view q = snapshot_view(captured.q);
                                  const iomx_view k = snapshot_view(captured.k);
                                  const iomx_view v = snapshot_view(captured.v);
                                  const iomx_view out = snapshot_view(captured.out);
                                  if (consume_submission_fault(SubmissionFault::sdpa_launch))
                                      return kInjectedDeviceError;
                                  // the library picks the kernel from the shapes, as its
                                  // workspace query did (a decode step and wide heads use none)
                                  return iomx_launch_sdpa(IOMX_DT_BF16, &q, &k, &v, &out, captured.a,
                                                          captured.L, scratch, scratch_bytes, 0, stream);
                              },
                              [this, &state, entries, lease, sequence](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_sdpa_entries(
                                          state.registry, entries, failed, proved);
                                  // Successful attention keeps its workspace range leased until
                                  // the caller observes the token (wait -> fence_through_sequence):
                                  // a second submission on the same range is then refused as
                                  // exhaustion whether or not the first has already finished
                                  // (src/shared/gpu_queue_operations.inl:1113-1147).  A failed
                                  // one, or one that leased nothing, releases at once.
                                  if (failed || lease.entry_id == 0 || !keep_until_observed(sequence, lease))
                                      detail::complete_workspace_lease(state, lease, proved);
                              });
                    } catch (...) {
                        state.registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        detail::complete_workspace_lease(state, lease, true);
                        throw;
                    }
                });
    }

    // ---- cache append / embedding / rope ----------------------------------------

    template <typename Snapshot>
    [[nodiscard]] static iomx_view snapshot_view(const Snapshot& s) {
        return make_view(s.native_handle, s.shape_dimensions(), s.plane_offset,
                         s.leading_plane_strides());
    }

    [[nodiscard]] WorkspaceRequirements cache_append_workspace_requirements(
            const CacheAppendRequest&) override {
        return {0, 1};
    }

    oid cache_append_impl(const CacheAppendRequest& request) override {
        const int code = transfer_code(request.source.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_cache_append(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const CacheAppendRequest& captured,
                             detail::BinaryEntryRegistration entries) {
                    auto& state = device_.registry_state();
                    const detail::WorkspaceLease lease = captured.workspace_lease;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  const iomx_view source = snapshot_view(captured.source);
                                  const iomx_view destination = snapshot_view(captured.destination);
                                  return iomx_launch_cache_append(code, &source, &destination,
                                                                  captured.a, stream);
                              },
                              [&state, entries, lease](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          state.registry, entries, failed, proved);
                                  detail::complete_workspace_lease(state, lease, proved);
                              });
                    } catch (...) {
                        state.registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        detail::complete_workspace_lease(state, lease, true);
                        throw;
                    }
                });
    }

    [[nodiscard]] WorkspaceRequirements rope_workspace_requirements(const RopeRequest& request) override {
        if (float_code(request.x.data_type) < 0) throw detail::UnsupportedOperation();
        return {0, 1};
    }

    oid rope_impl(const RopeRequest& request) override {
        const int code = float_code(request.x.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_rope(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const RopeRequest& captured,
                             detail::BinaryEntryRegistration entries) {
                    auto& registry = device_.registry_state().registry;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  const iomx_view x = snapshot_view(captured.x);
                                  const iomx_view out = snapshot_view(captured.out);
                                  return iomx_launch_rope(code, &x, &out, captured.a, captured.theta,
                                                          stream);
                              },
                              [&registry, entries](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          registry, entries, failed, proved);
                              });
                    } catch (...) {
                        registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        throw;
                    }
                });
    }

    // 32 bytes of caller-owned control scratch, 32-byte aligned: the first word is the
    // bounds status (docs/BACKEND_CONTRACT/embedding-lookup.md:178-201).
    [[nodiscard]] WorkspaceRequirements embedding_workspace_requirements_impl(
            const TensorView& table, const TensorView& indices, const TensorView&) override {
        if (transfer_code(table.spec().data_type) < 0) throw detail::UnsupportedOperation();
        const int index = static_cast<int>(indices.spec().data_type);
        if (index < static_cast<int>(DataType::I2) || index > static_cast<int>(DataType::U64))
            throw detail::UnsupportedOperation();
        return {32, 32};
    }

    oid embedding_impl(const EmbeddingRequest& request) override {
        const int code = transfer_code(request.table.spec.data_type);
        const int index_code = static_cast<int>(request.indices.spec.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_embedding(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code, index_code](std::uint64_t sequence, const EmbeddingRequest& captured,
                                         detail::BinaryEntryRegistration entries) {
                    auto& state = device_.registry_state();
                    const detail::WorkspaceLease lease = captured.workspace_lease;
                    try {
                        auto* control = static_cast<std::uint32_t*>(
                                detail::WorkspaceValidation::address(captured.workspace));
                        start(sequence,
                              [&captured, code, index_code, control](iomx_stream_t stream,
                                                                    std::uint32_t* cell) {
                                  const auto view_of = [](const CopyViewSnapshot& s) {
                                      return make_view(s.native_handle, s.spec.shape.dimensions(),
                                                       s.plane_offset, s.plane_strides);
                                  };
                                  const iomx_view table = view_of(captured.table);
                                  const iomx_view indices = view_of(captured.indices);
                                  const iomx_view out = view_of(captured.out);
                                  // status reset, gather, then exactly four bytes back to the host
                                  int status = iomx_launch_embedding(code, index_code, &table, &indices,
                                                                     &out, control, stream);
                                  if (status == IOMX_OK)
                                      status = consume_submission_fault(SubmissionFault::embedding_status_copy)
                                              ? kInjectedDeviceError
                                              : iomx_memcpy_d2h_async(cell, control, sizeof(*cell), stream);
                                  return status;
                              },
                              [&state, entries, lease](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          state.registry, entries, failed, proved);
                                  detail::complete_workspace_lease(state, lease, proved);
                              },
                              [](std::uint32_t status) -> std::exception_ptr {
                                  if (status == 0) return nullptr;
                                  return std::make_exception_ptr(std::invalid_argument(
                                          "MI355X embedding index is negative or out of range"));
                              });
                    } catch (...) {
                        state.registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        detail::complete_workspace_lease(state, lease, true);
                        throw;
                    }
                });
    }

    [[nodiscard]] WorkspaceRequirements silu_workspace_requirements_impl(
            const SiLURequest& request) override {
        if (float_code(request.x.data_type) < 0) throw detail::UnsupportedOperation();
        return {0, 1};
    }

    oid silu_impl(const SiLURequest& request) override {
        const int code = float_code(request.x.data_type);
        if (code < 0) throw detail::UnsupportedOperation();
        std::lock_guard<std::mutex> order(submission_mutex_);
        return submit_silu(
                request, device_.registry_state(), registry_queue_id_, pending_fence(),
                [this, code](std::uint64_t sequence, const SiLURequest& captured,
                             detail::BinaryEntryRegistration entries) {
                    auto& registry = device_.registry_state().registry;
                    try {
                        start(sequence,
                              [&captured, code](iomx_stream_t stream) {
                                  const auto view_of = [](const SiLUViewSnapshot& s) {
                                      return make_view(s.native_handle, s.shape_dimensions(),
                                                       s.plane_offset, s.leading_plane_strides());
                                  };
                                  const iomx_view x = view_of(captured.x);
                                  const iomx_view y = view_of(captured.y);
                                  if (consume_submission_fault(SubmissionFault::silu_launch))
                                      return kInjectedDeviceError;     // never reaches the kernel
                                  rocm_detail::silu_launch_count_for_testing.fetch_add(1);
                                  return iomx_launch_silu(code, &x, &y, stream);
                              },
                              [&registry, entries](bool failed, bool proved) {
                                  (void)detail::release_or_invalidate_binary_entries(
                                          registry, entries, failed, proved);
                              });
                    } catch (...) {
                        registry.remove_entries(std::span<const detail::EntryId>(
                                entries.entries.data(), entries.count));
                        throw;
                    }
                });
    }

    Mi355xDevice& device_;
    detail::QueueId registry_queue_id_;
    std::mutex submission_mutex_;
    iomx_stream_t stream_ = nullptr;
    std::vector<iomx_event_t> events_;
    std::uint32_t* status_cells_ = nullptr;
    std::uint32_t* cells_on_device_ = nullptr;   // the same cells at the address the device uses
    std::mutex mutex_;
    std::condition_variable cv_;
    std::vector<iomx_event_t> free_events_;
    std::deque<InFlight> in_flight_;
    std::atomic<std::size_t> pending_{0};   // in_flight_.size(), readable without the lock
    bool completer_sleeping_ = false;
    bool completing_ = false;
    std::uint32_t ticket_ = 0;          // last value handed to a completion word; never 0
    std::mutex observed_mutex_;
    std::map<std::uint64_t, detail::WorkspaceLease> unobserved_leases_;
    bool shutdown_ = false;
    std::thread completer_;
};

std::unique_ptr<Tensor> Mi355xDevice::create_tensor(const TensorSpec& spec) {
    return std::make_unique<Mi355xTensor>(spec, *this);
}

std::unique_ptr<RawWorkspace> Mi355xDevice::create_workspace(std::size_t bytes) {
    return std::make_unique<Mi355xWorkspace>(*this, bytes);
}

std::unique_ptr<DeviceOps> Mi355xDevice::create_ops() {
    return std::make_unique<Mi355xQueue>(*this);
}

}  // namespace

namespace rocm_detail {
void queue_resource_snapshot_for_testing(DeviceOps& queue, QueueResourceSnapshot& snapshot) {
    auto* mine = dynamic_cast<Mi355xQueue*>(&queue);
    if (mine == nullptr) throw std::invalid_argument("not an MI355X queue");
    mine->snapshot(snapshot);
}
std::size_t retained_queue_lease_count_for_testing(Device& device) {
    auto* mine = dynamic_cast<Mi355xDevice*>(&device);
    if (mine == nullptr) throw std::invalid_argument("not an MI355X device");
    return mine->retained_lease_count();
}
void reclaim_retained_queue_leases_for_testing(Device& device) {
    auto* mine = dynamic_cast<Mi355xDevice*>(&device);
    if (mine == nullptr) throw std::invalid_argument("not an MI355X device");
    mine->reclaim_retained_leases();
}
}  // namespace rocm_detail

// include/iom/rocm/device.hpp:22-24.  Configuration errors are reported before
// any native effect (include/iom/detail/gpu_arena_config.hpp:18-53).
std::unique_ptr<Device> make_rocm_device(std::uint32_t device_ordinal,
                                         DeviceMemoryConfig memory_config,
                                         QueueConfig queue_config) {
    const std::size_t arena = detail::valid_tensor_arena_bytes(memory_config.tensor_arena_bytes);
    (void)detail::standard_gpu_metadata_bytes(queue_config.max_in_flight_per_queue);
    return std::make_unique<Mi355xDevice>(device_ordinal, arena, queue_config);
}

}  // namespace iom
