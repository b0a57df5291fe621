// Test seams of the MI355X backend: host-side fault injection and resource counters, the
// counterpart of iom::rocm_detail in the reference's ROCm backend (src/rocm/copy.hpp:40-93,
// 521-543; src/rocm/driver.hpp:49-81).  Every fault is raised on the host -- a launch that is
// not made, a status that is replaced -- so no test makes the GPU itself fail.  The seams are
// always compiled in: an unarmed checkpoint is one relaxed atomic load.
#pragma once

#include <atomic>
#include <cstddef>

#include "iom/device.hpp"
#include "iom/iom.hpp"

namespace iom::rocm_detail {

// One-shot faults.  Where the reference has a seam of the same meaning the name is the
// reference's; `kernel_launch` stands where the reference fails its third per-plane launch
// (this backend makes one launch per operation).
enum class SubmissionFault {
    none,
    event_create,           // before acceptance: no completion resource -> negative OID (-5), no sequence used
    queue_event_create,     // queue construction: creating a completion event fails
    queue_stream_create,    // queue construction: creating the stream fails
    kernel_launch,          // after acceptance: the launch is not made and reports a device error
    embedding_status_copy,  // after the gather launch: the status word's copy to the host fails
    event_record,           // after the launch: recording the completion event fails
    stream_synchronize,     // queue destruction: the final proof of completion fails
    silu_launch,            // after acceptance, before the native SiLU launch
    sdpa_launch,            // after acceptance of an attention request
    event_record_unproved,  // as event_record, and the stream synchronisation that would prove the
                            // failed submission's work finished fails as well
};

void inject_submission_fault_for_testing(SubmissionFault fault) noexcept;
[[nodiscard]] bool consume_submission_fault(SubmissionFault fault) noexcept;

// Native resource lifecycle of queues and of the device arena.
extern std::atomic<std::size_t> event_create_count_for_testing;
extern std::atomic<std::size_t> event_destroy_count_for_testing;
extern std::atomic<std::size_t> stream_create_count_for_testing;
extern std::atomic<std::size_t> stream_destroy_count_for_testing;
extern std::atomic<std::size_t> device_allocation_count_for_testing;
extern std::atomic<std::size_t> device_free_count_for_testing;
// Which kernel an accepted submission reached.
extern std::atomic<std::size_t> linear_native_bf16_launch_count_for_testing;
extern std::atomic<std::size_t> linear_scalar_launch_count_for_testing;
extern std::atomic<std::size_t> silu_launch_count_for_testing;

// Fixed resources of one live queue: the C completion events created at construction and how
// many of them, and how many launched operations, are outstanding right now.
struct QueueResourceSnapshot {
    std::size_t events_total = 0;
    std::size_t events_in_use = 0;
    std::size_t operations_in_flight = 0;
};
void queue_resource_snapshot_for_testing(DeviceOps& queue, QueueResourceSnapshot& snapshot);

// Queue leases (stream, events, status cells, queue-count reservation) that a failed final
// synchronisation left at the device, and the attempt to prove them complete and reclaim them.
[[nodiscard]] std::size_t retained_queue_lease_count_for_testing(Device& device);
void reclaim_retained_queue_leases_for_testing(Device& device);

}  // namespace iom::rocm_detail
