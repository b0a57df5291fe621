// iomc_shim.cpp — a plain-C handle API over IOM's public C++ interface
// (iom::Device / iom::Tensor / iom::TensorView / iom::DeviceOps,
// include/iom/{device,tensor,iom}.hpp), so that Python tests can drive a
// backend exactly the way the reference's own conformance drivers do:
// create_tensor -> copy_from_host -> queue->add/mul/sub/copy/rmsnorm/silu ->
// wait -> copy_to_host.
//
// TEST INFRASTRUCTURE.  The file is compiled twice, against the reference's
// headers where they lie:
//   * with the reference CPU backend's own sources -> oracle/_ref/libiom_ref.so
//     (factory: iom::make_cpu_device, include/iom/cpu/device.hpp:19-20);
//   * -DIOMC_WITH_MI355X with this repository's backend ->
//     iom_amd/lib/libiom_mi355x_shim.so (factory: iom::make_rocm_device,
//     include/iom/rocm/device.hpp:22-24).
// It holds no arithmetic of its own.
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <exception>
#include <memory>
#include <new>
#include <span>
#include <stdexcept>
#include <string>
#include <vector>

#include "iom/alloc.hpp"
#include "iom/cpu/device.hpp"
#include "iom/device.hpp"
#include "iom/iom.hpp"
#include "iom/tensor.hpp"
#include "src/iom_internal.hpp"  // iom::detail::UnsupportedOperation
#ifndef IOMC_WITH_MI355X
// The reference's own backend-free attention reference and fixture corpus.
#include "test/backend/backend_conformance_sdpa_reference.hpp"
#endif
#ifdef IOMC_WITH_MI355X
#include "iom/rocm/device.hpp"
#include "../iom_amd/host/mi355x_testing.hpp"  // fault injection and resource counters
#endif

namespace {

thread_local std::string g_error;

// Error classes mirror the negative OID mapping of src/device_ops.cpp:422-439.
int classify(const std::exception_ptr& failure) {
    try {
        std::rethrow_exception(failure);
    } catch (const iom::detail::UnsupportedOperation& e) {
        g_error = std::string("unsupported: ") + e.what();
        return -2;
    } catch (const std::bad_alloc& e) {
        g_error = std::string("bad_alloc: ") + e.what();
        return -4;
    } catch (const std::overflow_error& e) {
        g_error = std::string("overflow_error: ") + e.what();
        return -3;
    } catch (const std::invalid_argument& e) {
        g_error = std::string("invalid_argument: ") + e.what();
        return -1;
    } catch (const std::out_of_range& e) {
        g_error = std::string("out_of_range: ") + e.what();
        return -7;
    } catch (const std::exception& e) {
        g_error = std::string("exception: ") + e.what();
        return -5;
    } catch (...) {
        g_error = "unknown failure";
        return -6;
    }
}

class HeapAllocator final : public iom::Allocator {
public:
    void* alloc(std::size_t size) override {
        return ::operator new(size, std::align_val_t(64));
    }
    void free(void* buffer) override {
        ::operator delete(buffer, std::align_val_t(64));
    }
    void reset() override {}
};

}  // namespace

struct iomc_device {
    HeapAllocator allocator;
    std::unique_ptr<iom::Device> device;
};
struct iomc_tensor {
    std::unique_ptr<iom::Tensor> tensor;
};
struct iomc_view {
    iom::TensorView view;
};
struct iomc_queue {
    std::unique_ptr<iom::DeviceOps> ops;
};
struct iomc_workspace {
    std::unique_ptr<iom::RawWorkspace> workspace;
};

namespace {

template <typename F>
auto guarded(F&& body, decltype(body()) fallback) -> decltype(body()) {
    try {
        return body();
    } catch (...) {
        (void)classify(std::current_exception());
        return fallback;
    }
}

template <typename F>
int guarded_status(F&& body) {
    try {
        body();
        return 0;
    } catch (...) {
        return classify(std::current_exception());
    }
}

// Host transfers on accelerator backends need a caller workspace of the
// queried size (src/rocm/device_tensor.cpp:136-143); the CPU backend reports
// {0,1}.
std::unique_ptr<iom::RawWorkspace> transfer_workspace(
        iom::Device& device, const iom::WorkspaceRequirements& need) {
    if (need.bytes == 0) return nullptr;
    return device.create_workspace(need.bytes);
}

}  // namespace

extern "C" {

const char* iomc_last_error() { return g_error.c_str(); }

iomc_device* iomc_cpu_device_create(std::size_t max_in_flight) {
    return guarded([&]() -> iomc_device* {
        auto holder = std::make_unique<iomc_device>();
        holder->device = iom::make_cpu_device(
                holder->allocator, iom::QueueConfig{max_in_flight});
        return holder.release();
    }, nullptr);
}

#ifdef IOMC_WITH_MI355X
iomc_device* iomc_mi355x_device_create(
        std::uint32_t ordinal, std::size_t arena_bytes,
        std::size_t max_in_flight) {
    return guarded([&]() -> iomc_device* {
        auto holder = std::make_unique<iomc_device>();
        holder->device = iom::make_rocm_device(
                ordinal, iom::DeviceMemoryConfig{arena_bytes},
                iom::QueueConfig{max_in_flight});
        return holder.release();
    }, nullptr);
}
#endif

void iomc_device_destroy(iomc_device* device) { delete device; }

int iomc_device_backend_kind(const iomc_device* device) {
    return static_cast<int>(device->device->backend_kind());
}

// Device::supported_data_types() (include/iom/device.hpp:57-131): writes up to
// `capacity` leaf codes in the advertised order and returns the full count.
std::uint32_t iomc_device_supported_types(const iomc_device* device, int* codes, std::uint32_t capacity) {
    const auto types = device->device->supported_data_types();
    for (std::uint32_t i = 0; i < types.size() && i < capacity; ++i) codes[i] = static_cast<int>(types[i]);
    return static_cast<std::uint32_t>(types.size());
}

iomc_tensor* iomc_tensor_create(
        iomc_device* device, int dtype, std::uint32_t rank,
        const std::uint64_t* dims) {
    return guarded([&]() -> iomc_tensor* {
        std::vector<std::size_t> shape(dims, dims + rank);
        iom::TensorSpec spec{
                iom::TensorShape{std::move(shape)},
                static_cast<iom::DataType>(dtype)};
        auto holder = std::make_unique<iomc_tensor>();
        holder->tensor = device->device->create_tensor(spec);
        return holder.release();
    }, nullptr);
}

void iomc_tensor_destroy(iomc_tensor* tensor) { delete tensor; }

iomc_view* iomc_tensor_view(iomc_tensor* tensor) {
    return guarded([&]() -> iomc_view* {
        return new iomc_view{tensor->tensor->view()};
    }, nullptr);
}

void iomc_view_destroy(iomc_view* view) { delete view; }

iomc_view* iomc_view_slice(
        const iomc_view* view, std::size_t dim, std::size_t first,
        std::size_t count, std::size_t step) {
    return guarded([&]() -> iomc_view* {
        return new iomc_view{view->view.slice(dim, first, count, step)};
    }, nullptr);
}

iomc_view* iomc_view_select(
        const iomc_view* view, std::size_t dim, std::size_t index) {
    return guarded([&]() -> iomc_view* {
        return new iomc_view{view->view.select(dim, index)};
    }, nullptr);
}

iomc_view* iomc_view_permute(
        const iomc_view* view, const std::uint64_t* order, std::size_t count) {
    return guarded([&]() -> iomc_view* {
        std::vector<std::size_t> axes(order, order + count);
        return new iomc_view{view->view.permute(axes)};
    }, nullptr);
}

iomc_view* iomc_view_reshape_leading(
        const iomc_view* view, const std::uint64_t* dims, std::size_t count) {
    return guarded([&]() -> iomc_view* {
        std::vector<std::size_t> leading(dims, dims + count);
        return new iomc_view{view->view.reshape_leading(leading)};
    }, nullptr);
}

std::uint32_t iomc_view_rank(const iomc_view* view) {
    return static_cast<std::uint32_t>(view->view.spec().shape.rank());
}

void iomc_view_describe(
        const iomc_view* view, std::uint64_t* dims, std::uint64_t* plane_offset,
        std::uint64_t* plane_strides) {
    const auto shape = view->view.spec().shape.dimensions();
    for (std::size_t i = 0; i < shape.size(); ++i) dims[i] = shape[i];
    *plane_offset = view->view.plane_offset();
    const auto strides = view->view.plane_strides();
    for (std::size_t i = 0; i < strides.size(); ++i) plane_strides[i] = strides[i];
}

std::uint64_t iomc_view_logical_nbytes(const iomc_view* view) {
    return guarded([&]() -> std::uint64_t {
        return view->view.spec().logical_nbytes();
    }, 0);
}

std::uint64_t iomc_view_tiled_nbytes(const iomc_view* view) {
    return guarded([&]() -> std::uint64_t {
        return view->view.spec().tiled_storage_nbytes();
    }, 0);
}

// Raw owner storage: host memory on the CPU backend, device memory on an
// accelerator backend (include/iom/tensor.hpp:290-291).
void* iomc_view_native_handle(iomc_view* view) {
    return view->view.native_handle();
}

int iomc_view_from_host(
        iomc_device* device, iomc_view* view, const void* bytes,
        std::size_t nbytes) {
    return guarded_status([&] {
        auto workspace = transfer_workspace(
                *device->device,
                view->view.copy_from_host_workspace_requirements());
        const std::span<const std::byte> source(
                static_cast<const std::byte*>(bytes), nbytes);
        if (workspace) view->view.copy_from_host(source, workspace->view());
        else view->view.copy_from_host(source);
    });
}

int iomc_view_to_host(
        iomc_device* device, const iomc_view* view, void* bytes,
        std::size_t nbytes) {
    return guarded_status([&] {
        auto workspace = transfer_workspace(
                *device->device,
                view->view.copy_to_host_workspace_requirements());
        const std::span<std::byte> destination(
                static_cast<std::byte*>(bytes), nbytes);
        if (workspace) view->view.copy_to_host(destination, workspace->view());
        else view->view.copy_to_host(destination);
    });
}

iomc_queue* iomc_queue_create(iomc_device* device) {
    return guarded([&]() -> iomc_queue* {
        auto holder = std::make_unique<iomc_queue>();
        holder->ops = device->device->create_ops();
        return holder.release();
    }, nullptr);
}

void iomc_queue_destroy(iomc_queue* queue) { delete queue; }

// op: 0 add, 1 mul, 2 sub, 3 div (order of scalar_binary_codec.hpp:9).
std::int64_t iomc_binary(
        iomc_queue* queue, int op, const iomc_view* lhs, const iomc_view* rhs,
        iomc_view* out) {
    switch (op) {
        case 0: return queue->ops->add(lhs->view, rhs->view, out->view);
        case 1: return queue->ops->mul(lhs->view, rhs->view, out->view);
        case 2: return queue->ops->sub(lhs->view, rhs->view, out->view);
        case 3: return queue->ops->div(lhs->view, rhs->view, out->view);
        default: return -1;
    }
}

std::int64_t iomc_copy(
        iomc_queue* queue, const iomc_view* source, iomc_view* destination) {
    return queue->ops->copy(source->view, destination->view);
}

std::int64_t iomc_rmsnorm(
        iomc_queue* queue, const iomc_view* x, const iomc_view* scale,
        iomc_view* out, float eps) {
    return queue->ops->rmsnorm(x->view, scale->view, out->view, eps);
}

std::int64_t iomc_silu(iomc_queue* queue, const iomc_view* x, iomc_view* y) {
    return queue->ops->silu(x->view, y->view);
}

// Full attention through the public facade; the softmax stage has no public
// entry of its own (docs/BACKEND_CONTRACT/scaled-dot-product-attention.md:9-10).
std::int64_t iomc_sdpa(
        iomc_device* device, iomc_queue* queue, const iomc_view* q,
        const iomc_view* k, const iomc_view* v, iomc_view* out, std::size_t a,
        std::size_t L) {
    try {
        const iom::WorkspaceRequirements need =
                queue->ops->sdpa_workspace_requirements(
                        q->view, k->view, v->view, out->view, a, L);
        if (need.bytes == 0) {
            return queue->ops->sdpa(q->view, k->view, v->view, out->view, a, L);
        }
        auto workspace = device->device->create_workspace(need.bytes);
        const iom::oid token = queue->ops->sdpa(
                q->view, k->view, v->view, out->view, a, L, workspace->view());
        if (token > 0) queue->ops->wait(token);
        return token;
    } catch (...) {
        return classify(std::current_exception());
    }
}

// out[b,r,o] = sum_i x[b,s+r,i] * w[o,i], ordinary or head planar
// (docs/BACKEND_CONTRACT/linear-projections.md:20-31).
std::int64_t iomc_linear(
        iomc_queue* queue, const iomc_view* x, const iomc_view* w, iomc_view* out, std::size_t s,
        std::size_t R, int head_planar, std::size_t H, std::size_t D) {
    return queue->ops->linear(
            x->view, w->view, out->view, s, R,
            head_planar ? iom::LinearOutputLayout::head_planar : iom::LinearOutputLayout::ordinary,
            H, D);
}

// destination[..., h, a + r, d] = source[..., h, r, d] (include/iom/iom.hpp:171-182).
std::int64_t iomc_cache_append(
        iomc_queue* queue, const iomc_view* source, iomc_view* destination, std::size_t a) {
    return queue->ops->cache_append(source->view, destination->view, a);
}

// Split-half rotary position encoding (include/iom/iom.hpp:343-357).
std::int64_t iomc_rope(
        iomc_queue* queue, const iomc_view* x, iomc_view* out, std::size_t a, double theta) {
    return queue->ops->rope(x->view, out->view, a, theta);
}

// out[b, r, f] = table[indices[b, 0, r], f] (include/iom/iom.hpp:188-223).  A backend
// that asks for control scratch gets a workspace of exactly that size; the call then
// waits so the scratch can be released, and reports the wait's outcome apart from the
// submission's (0 = completed, negative = the retained failure's class).
std::int64_t iomc_embedding(
        iomc_device* device, iomc_queue* queue, const iomc_view* table,
        const iomc_view* indices, iomc_view* out, int* wait_status) {
    if (wait_status) *wait_status = 0;
    try {
        const iom::WorkspaceRequirements need =
                queue->ops->embedding_workspace_requirements(
                        table->view, indices->view, out->view);
        std::unique_ptr<iom::RawWorkspace> workspace;
        iom::oid token;
        if (need.bytes == 0) {
            token = queue->ops->embedding(table->view, indices->view, out->view);
        } else {
            workspace = device->device->create_workspace(need.bytes);
            token = queue->ops->embedding(
                    table->view, indices->view, out->view, workspace->view());
        }
        if (token > 0) {
            try {
                queue->ops->wait(token);
            } catch (...) {
                if (wait_status) *wait_status = static_cast<int>(classify(std::current_exception()));
            }
        }
        return token;
    } catch (...) {
        return classify(std::current_exception());
    }
}

#ifndef IOMC_WITH_MI355X
// The fixed attention fixtures of test/backend/backend_conformance_sdpa_reference.hpp
// (sdpa_reference_cases, :1267-1299), their expected values (evaluate, :988) and the
// comparison rule (matches, :1232-1259), for writing golden vectors.
namespace {
const std::vector<iom_conformance::SdpaReferenceCase>& sdpa_cases() {
    static const std::vector<iom_conformance::SdpaReferenceCase> cases =
            iom_conformance::sdpa_reference_cases(iom::DataType::BF16);
    return cases;
}
}  // namespace

int iomc_sdpa_case_count() { return static_cast<int>(sdpa_cases().size()); }

// info: kind, leading rank, 4 leading dimensions, Hq, Hkv, R, D, C, a, L, padding salt
int iomc_sdpa_case_info(int index, std::uint64_t* info, char* label, std::size_t label_size) {
    if (index < 0 || index >= iomc_sdpa_case_count()) return -1;
    const auto& c = sdpa_cases()[static_cast<std::size_t>(index)];
    if (c.leading_dimensions.size() > 4) return -1;
    info[0] = static_cast<std::uint64_t>(c.kind);
    info[1] = c.leading_dimensions.size();
    for (std::size_t i = 0; i < 4; ++i) info[2 + i] = i < c.leading_dimensions.size() ? c.leading_dimensions[i] : 1;
    info[6] = c.hq; info[7] = c.hkv; info[8] = c.rows; info[9] = c.head_dim;
    info[10] = c.capacity; info[11] = c.position; info[12] = c.length;
    info[13] = c.physical_padding_salt;
    info[14] = c.q_bits.size(); info[15] = c.k_bits.size(); info[16] = c.v_bits.size();
    const std::string text = iom_conformance::sdpa_reference_case_label(c);
    std::strncpy(label, text.c_str(), label_size - 1);
    label[label_size - 1] = 0;
    return 0;
}

int iomc_sdpa_case_data(int index, std::uint16_t* q, std::uint16_t* k, std::uint16_t* v) {
    if (index < 0 || index >= iomc_sdpa_case_count()) return -1;
    const auto& c = sdpa_cases()[static_cast<std::size_t>(index)];
    for (std::size_t i = 0; i < c.q_bits.size(); ++i) q[i] = static_cast<std::uint16_t>(c.q_bits[i]);
    for (std::size_t i = 0; i < c.k_bits.size(); ++i) k[i] = static_cast<std::uint16_t>(c.k_bits[i]);
    for (std::size_t i = 0; i < c.v_bits.size(); ++i) v[i] = static_cast<std::uint16_t>(c.v_bits[i]);
    return 0;
}

// Expected output [B..., R, Hq*D] row-major: raw bits and value class per element.
std::int64_t iomc_sdpa_case_expected(int index, std::uint16_t* bits, std::uint8_t* classes, std::size_t capacity) {
    if (index < 0 || index >= iomc_sdpa_case_count()) return -1;
    try {
        const auto values = iom_conformance::evaluate(sdpa_cases()[static_cast<std::size_t>(index)]);
        if (values.size() > capacity) return -static_cast<std::int64_t>(values.size());
        for (std::size_t i = 0; i < values.size(); ++i) {
            bits[i] = static_cast<std::uint16_t>(values[i].bits);
            classes[i] = static_cast<std::uint8_t>(values[i].value_class);
        }
        return static_cast<std::int64_t>(values.size());
    } catch (...) {
        return classify(std::current_exception());
    }
}

int iomc_sdpa_matches(std::uint16_t actual, std::uint16_t expected_bits, std::uint8_t expected_class) {
    iom_conformance::SdpaReferenceValue expected;
    expected.bits = expected_bits;
    expected.value_class = static_cast<iom_conformance::SdpaReferenceClass>(expected_class);
    return iom_conformance::matches(iom::DataType::BF16, static_cast<std::uint64_t>(actual), expected) ? 1 : 0;
}
#endif

int iomc_wait(iomc_queue* queue, std::int64_t token) {
    return guarded_status([&] { queue->ops->wait(token); });
}

// ---- submissions that do not wait, with the workspace owned by the caller ---------------
// (what the conformance drivers do when they test lifetimes: drop an owner while its
// operation is still in flight, test/rocm/test_rocm_conformance.cpp)

iomc_workspace* iomc_workspace_create(iomc_device* device, std::size_t bytes) {
    return guarded([&]() -> iomc_workspace* {
        auto holder = std::make_unique<iomc_workspace>();
        holder->workspace = device->device->create_workspace(bytes);
        return holder.release();
    }, nullptr);
}

void iomc_workspace_destroy(iomc_workspace* workspace) { delete workspace; }

std::int64_t iomc_sdpa_workspace_bytes(
        iomc_queue* queue, const iomc_view* q, const iomc_view* k, const iomc_view* v,
        const iomc_view* out, std::size_t a, std::size_t L) {
    try {
        return static_cast<std::int64_t>(queue->ops->sdpa_workspace_requirements(
                q->view, k->view, v->view, out->view, a, L).bytes);
    } catch (...) {
        return classify(std::current_exception());
    }
}

std::int64_t iomc_sdpa_submit(
        iomc_queue* queue, const iomc_view* q, const iomc_view* k, const iomc_view* v,
        iomc_view* out, std::size_t a, std::size_t L, iomc_workspace* workspace) {
    if (workspace == nullptr) return queue->ops->sdpa(q->view, k->view, v->view, out->view, a, L);
    return queue->ops->sdpa(q->view, k->view, v->view, out->view, a, L, workspace->workspace->view());
}

std::int64_t iomc_embedding_submit(
        iomc_queue* queue, const iomc_view* table, const iomc_view* indices, iomc_view* out,
        iomc_workspace* workspace) {
    if (workspace == nullptr) return queue->ops->embedding(table->view, indices->view, out->view);
    return queue->ops->embedding(table->view, indices->view, out->view, workspace->workspace->view());
}

std::int64_t iomc_embedding_workspace_bytes(
        iomc_queue* queue, const iomc_view* table, const iomc_view* indices, const iomc_view* out) {
    try {
        return static_cast<std::int64_t>(queue->ops->embedding_workspace_requirements(
                table->view, indices->view, out->view).bytes);
    } catch (...) {
        return classify(std::current_exception());
    }
}

#ifdef IOMC_WITH_MI355X
// ---- the MI355X backend's test seams (iom_amd/host/mi355x_testing.hpp) -------------------

// fault: numeric value of iom::rocm_detail::SubmissionFault
void iomc_inject_fault(int fault) {
    iom::rocm_detail::inject_submission_fault_for_testing(
            static_cast<iom::rocm_detail::SubmissionFault>(fault));
}

// which: 0 event create, 1 event destroy, 2 stream create, 3 stream destroy, 4 device
// allocations, 5 device frees, 6 native BF16 linear launches, 7 scalar linear launches, 8 SiLU launches
std::uint64_t iomc_test_counter(int which) {
    using namespace iom::rocm_detail;
    switch (which) {
        case 0: return event_create_count_for_testing.load();
        case 1: return event_destroy_count_for_testing.load();
        case 2: return stream_create_count_for_testing.load();
        case 3: return stream_destroy_count_for_testing.load();
        case 4: return device_allocation_count_for_testing.load();
        case 5: return device_free_count_for_testing.load();
        case 6: return linear_native_bf16_launch_count_for_testing.load();
        case 7: return linear_scalar_launch_count_for_testing.load();
        case 8: return silu_launch_count_for_testing.load();
        default: return ~std::uint64_t{0};
    }
}

int iomc_queue_snapshot(iomc_queue* queue, std::uint64_t* out3) {
    return guarded_status([&] {
        iom::rocm_detail::QueueResourceSnapshot snapshot;
        iom::rocm_detail::queue_resource_snapshot_for_testing(*queue->ops, snapshot);
        out3[0] = snapshot.events_total;
        out3[1] = snapshot.events_in_use;
        out3[2] = snapshot.operations_in_flight;
    });
}

std::int64_t iomc_retained_leases(iomc_device* device) {
    return guarded([&]() -> std::int64_t {
        return static_cast<std::int64_t>(
                iom::rocm_detail::retained_queue_lease_count_for_testing(*device->device));
    }, std::int64_t{-1});
}

void iomc_reclaim_leases(iomc_device* device) {
    (void)guarded_status([&] {
        iom::rocm_detail::reclaim_retained_queue_leases_for_testing(*device->device);
    });
}
#endif  // IOMC_WITH_MI355X

}  // extern "C"
