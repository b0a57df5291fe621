// Runs IOM's own backend-agnostic conformance scenarios against this repository's backend.
//
// The scenarios are the reference's: test/backend/backend_conformance_*.hpp, included from where
// they lie (the build adds <reference>/test and <reference> to the include path; nothing of them
// is kept in this repository).  This file only does what a backend's own driver does for them
// (test/rocm/test_rocm_conformance.cpp is the one for the reference's ROCm backend): it makes the
// devices -- the reference CPU backend as the expected side, iom::make_rocm_device as the
// candidate, a second instance as the foreign device --, hands over a storage oracle that reads
// and writes raw tiled device memory, names the fault seam a scenario may arm, and calls the
// shared runner.  Every assertion that decides pass or fail is the reference's.
//
// The candidate is reached through the same factory symbol a consumer of libiom links against;
// raw device memory is reached through the C ABI (iomx_memcpy_*), never through a HIP header.
#include <doctest/doctest.h>

#include <array>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <memory>
#include <new>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <unordered_set>
#include <vector>

#include "backend/backend_conformance_common.hpp"
#include "backend/backend_conformance_rope.hpp"
#include "backend/backend_conformance_rope_contract.hpp"
#include "backend/backend_conformance_cache_append.hpp"
#include "backend/backend_conformance_embedding.hpp"
#include "backend/backend_conformance_linear.hpp"
#include "backend/backend_conformance_other.hpp"
#include "backend/backend_conformance_rmsnorm.hpp"
#include "backend/backend_conformance_silu.hpp"
#include "backend/backend_conformance_add_gpu.hpp"
#include "backend/backend_conformance_sdpa.hpp"
#include "iom/alloc.hpp"
#include "iom/cpu/device.hpp"
#include "iom/gpu_algorithm.hpp"
#include "iom/rocm/device.hpp"

#include "iomx.h"
#include "mi355x_testing.hpp"

namespace {

namespace conf = iom_conformance;
namespace seams = iom::rocm_detail;

// The arena the reference's driver gives every fixture (test/rocm/test_rocm_conformance.cpp:55-59):
// three 8192x4096 F32 tensors plus one quarantined operand.
constexpr std::size_t kArenaBytes = 640u * 1024 * 1024;

// Host allocator for the CPU reference device of the scenarios that watch allocator traffic: an
// allocation or a release while the gate is armed (inside a transfer or an operation) is a failure.
class GatedHostAllocator final : public iom::Allocator {
public:
    explicit GatedHostAllocator(const conf::TrafficGate& gate) : gate_(gate) {}

    void* alloc(std::size_t size) override {
        CHECK_MESSAGE(!gate_.armed(), "host storage allocated while the traffic gate was armed");
        void* pointer = ::operator new(size, std::align_val_t(32));
        live_.insert(pointer);
        return pointer;
    }

    void free(void* buffer) override {
        CHECK_MESSAGE(!gate_.armed(), "host storage released while the traffic gate was armed");
        REQUIRE_MESSAGE(live_.erase(buffer) == 1, "released an address that was never handed out");
        ::operator delete(buffer, std::align_val_t(32));
    }

    void reset() override {}

private:
    const conf::TrafficGate& gate_;
    std::unordered_set<void*> live_;
};

// Raw tiled storage of an owner, byte for byte, through the C ABI.  native_handle() of any view is
// its owner's base address; the scenario sets the owner's spec before each use.
class RawStorageOracle final : public conf::AcceleratorStorageOracle {
public:
    void seed(iom::TensorView& view, std::span<const std::byte> encoded) override {
        const std::size_t bytes = owner_spec().tiled_storage_nbytes();
        REQUIRE_EQ(encoded.size(), bytes);
        REQUIRE_EQ(iomx_device_synchronize(), IOMX_OK);
        REQUIRE_EQ(iomx_memcpy_h2d(view.native_handle(), encoded.data(), bytes), IOMX_OK);
        REQUIRE_EQ(iomx_device_synchronize(), IOMX_OK);
    }

    [[nodiscard]] std::vector<std::byte> observe(const iom::TensorView& view) const override {
        const std::size_t bytes = owner_spec().tiled_storage_nbytes();
        std::vector<std::byte> result(bytes);
        REQUIRE_EQ(iomx_device_synchronize(), IOMX_OK);
        REQUIRE_EQ(iomx_memcpy_d2h(result.data(), view.native_handle(), bytes), IOMX_OK);
        return result;
    }
};

// The three devices of a scenario.  The CPU reference draws from a linear host arena unless the
// scenario watches allocator traffic.
struct Fixture {
    explicit Fixture(std::size_t reference_bytes = 64u * 1024 * 1024)
            : storage(reference_bytes),
              linear(storage.data(), storage.size()),
              reference(iom::make_cpu_device(linear)),
              candidate(iom::make_rocm_device(0, iom::DeviceMemoryConfig{kArenaBytes})),
              foreign(iom::make_rocm_device(0, iom::DeviceMemoryConfig{kArenaBytes})) {}

    [[nodiscard]] conf::ConformanceDevices devices() const {
        return conf::ConformanceDevices{*reference, *candidate, *foreign};
    }

    conf::TrafficGate gate;
    std::vector<std::byte> storage;
    iom::LinearAllocator linear;
    std::unique_ptr<iom::Device> reference;
    std::unique_ptr<iom::Device> candidate;
    std::unique_ptr<iom::Device> foreign;
};

[[nodiscard]] std::unique_ptr<iom::Device> make_candidate() {
    return iom::make_rocm_device(0, iom::DeviceMemoryConfig{kArenaBytes});
}

void arm(seams::SubmissionFault fault) { seams::inject_submission_fault_for_testing(fault); }
void disarm() { seams::inject_submission_fault_for_testing(seams::SubmissionFault::none); }

}  // namespace

// ---- capability --------------------------------------------------------------------------------

TEST_CASE("MI355X: supported_data_types is the standard 23-entry span") {
    const auto candidate = make_candidate();
    CHECK_EQ(candidate->backend_kind(), iom::BackendKind::ROCM);
    conf::require_standard_capabilities(candidate->supported_data_types());
}

// ---- storage, host transfers, copies -----------------------------------------------------------

TEST_CASE("MI355X: storage and host transfers for every leaf type") {
    Fixture f;
    conf::run_storage_and_transfer_conformance(
            f.devices(), f.candidate->supported_data_types(), &f.gate);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: storage oracle tells a perturbed tile map from the true one") {
    Fixture f;
    const std::span<const iom::DataType> one_type = f.candidate->supported_data_types().subspan(0, 1);
    RawStorageOracle direct;
    conf::PermutingStorageOracle perturbed(direct, conf::swap_first_adjacent_slots);
    CHECK_FALSE(conf::run_storage_oracle_conformance(
            f.devices(), one_type, perturbed, &f.gate, false, false));
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: raw tiled storage of every leaf width and padded shape") {
    Fixture f;
    RawStorageOracle oracle;
    REQUIRE(conf::run_storage_oracle_conformance(
            f.devices(), f.candidate->supported_data_types(), oracle, &f.gate));
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: asynchronous copies against the CPU reference") {
    Fixture f;
    RawStorageOracle oracle;
    conf::run_async_copy_conformance(
            f.devices(), f.candidate->supported_data_types(), &f.gate, &oracle);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: copy validation fails before writes and sequences") {
    Fixture f(16u * 1024 * 1024);
    conf::run_copy_error_conformance(f.devices(), f.candidate->supported_data_types(), &f.gate);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: transfer failures keep metadata and ownership") {
    Fixture f(16u * 1024 * 1024);
    conf::run_transfer_error_conformance(f.devices(), f.candidate->supported_data_types(), &f.gate);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: sub-byte odd-length host reads") {
    const auto candidate = make_candidate();
    constexpr std::uint64_t salt = 0x180001ull;
    for (const iom::DataType type :
         {iom::DataType::I2, iom::DataType::F6_E2M3, iom::DataType::F6_E3M2}) {
        const iom::TensorSpec spec{iom::TensorShape{std::vector<std::size_t>{1, 17}}, type};
        const std::vector<std::byte> expected = conf::encode_logical(spec, salt);
        auto tensor = candidate->create_tensor(spec);
        conf::copy_from_host(tensor->view(), expected);
        conf::require_logical_bytes(tensor->view(), expected, "odd-length sub-byte host read");
    }
}

// ---- queue lifetime and capability -------------------------------------------------------------

TEST_CASE("MI355X: deferred queue lifetime and stability") {
    conf::TrafficGate gate;
    const auto candidate = make_candidate();
    conf::run_lifetime_conformance(*candidate, candidate->supported_data_types(), &gate);
    CHECK_FALSE(gate.armed());
}

TEST_CASE("MI355X: compute methods reject capability without submitting") {
    conf::TrafficGate gate;
    const auto candidate = make_candidate();
    conf::run_compute_capability_conformance(
            *candidate, candidate->supported_data_types(), &gate, "MI355X", true, true, true);
    CHECK_FALSE(gate.armed());
}

TEST_CASE("MI355X: rank-eight owners accepted, rank nine rejected") {
    const auto candidate = make_candidate();
    conf::run_accelerator_rank_boundary_conformance(*candidate);
}

// ---- binary operations -------------------------------------------------------------------------

TEST_CASE("MI355X: ADD MUL SUB DIV on the real queue, values, mappings and exact aliases") {
    const auto candidate = make_candidate();
    for (const auto operation : {conf::BinaryOperation::add, conf::BinaryOperation::mul,
                                 conf::BinaryOperation::sub, conf::BinaryOperation::div}) {
        CAPTURE(static_cast<int>(operation));
        conf::run_gpu_eltwise_conformance(*candidate, operation);
        conf::run_gpu_eltwise_mapping_conformance(*candidate, operation);
        conf::run_gpu_exact_alias_conformance(*candidate, operation);
    }
}

TEST_CASE("MI355X: binary rank boundary") {
    const auto candidate = make_candidate();
    conf::run_binary_rank_boundary_conformance(*candidate);
}

// ---- RMSNorm, SiLU -----------------------------------------------------------------------------

TEST_CASE("MI355X: RMSNorm reference, admission and lifetime") {
    Fixture f;
    RawStorageOracle oracle;
    conf::RmsNormConformanceConfig config{f.devices(), conf::kRmsNormAllLeafSpan, &f.gate, &oracle};
    // The completion event is recorded right after the launch; failing that record is an
    // accepted submission with a retained failure, which is what the scenario asks of the seam.
    config.native_failure = conf::RmsNormNativeFailureSeam{
            [] { arm(seams::SubmissionFault::event_record); },
            [] { disarm(); },
            "rocm_detail::SubmissionFault::event_record",
            {}};
    conf::run_rmsnorm_conformance(config);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: SiLU reference, admission and lifetime") {
    Fixture f;
    RawStorageOracle oracle;
    conf::SiluConformanceConfig config{
            f.devices(),
            conf::kSiluRocmExpectedSupported,
            &f.gate,
            &oracle,
            conf::SiluNativeFailureSeam{
                    [] { arm(seams::SubmissionFault::silu_launch); },
                    [] { disarm(); },
                    "rocm_detail::SubmissionFault::silu_launch",
                    {}}};
    conf::run_silu_conformance(config);
    CHECK_FALSE(f.gate.armed());
}

// ---- the operations either side of the hot path -------------------------------------------------

TEST_CASE("MI355X: cache append reference, admission, ordering and lifetime") {
    conf::TrafficGate gate;
    GatedHostAllocator reference_allocator{gate};
    const auto reference = iom::make_cpu_device(reference_allocator);
    const auto candidate = make_candidate();
    const auto foreign = make_candidate();
    const conf::ConformanceDevices devices{*reference, *candidate, *foreign};
    RawStorageOracle oracle;
    // One launch serves a whole append here, so the accepted failure the scenario asks for is that
    // launch reporting a device error.
    const conf::CacheAppendFaultSeam fault_seam{
            [](iom::DeviceOps&) { arm(seams::SubmissionFault::kernel_launch); }};
    const conf::CacheAppendConformanceConfig config{
            devices, candidate->supported_data_types(), &oracle, fault_seam, {}, &gate};
    conf::run_cache_append_conformance(config);
    disarm();
    CHECK_FALSE(gate.armed());
}

// Every payload and index leaf, a 32-byte control workspace whose first word is the status
// (docs/BACKEND_CONTRACT/embedding.md; the same declaration the reference's accelerator drivers
// make, test/rocm/test_rocm_conformance.cpp:862-869).
constexpr conf::EmbeddingDeclaration kEmbeddingDeclaration{
        conf::kEmbeddingPayloadSpan, conf::kEmbeddingIdSpan, conf::kEmbeddingPayloadSpan,
        conf::kEmbeddingIdSpan, iom::WorkspaceRequirements{32, 32}};

TEST_CASE("MI355X: embedding lookup reference, admission and lifetime") {
    Fixture f;
    RawStorageOracle oracle;
    conf::run_embedding_conformance(f.devices(), kEmbeddingDeclaration, &f.gate, &oracle);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: RoPE reference, admission and lifetime") {
    const auto candidate = make_candidate();
    RawStorageOracle oracle;
    conf::rope_reference::run_rope_conformance(
            *candidate, conf::rope_reference::kRopeRocmExpectedSupported, oracle);
}

// All 21 numeric leaves are queued; BF16 runs on the matrix cores straight from the tiled operands
// and, like the twenty scalar leaves, asks for no caller workspace.
const conf::LinearDeclaration kLinearDeclaration{
        conf::kLinearLeafSpan,
        conf::kLinearScalarLeafSpan,
        conf::kLinearNativeBf16Span,
        conf::kLinearLeafSpan,
        {},
        conf::LinearWorkspacePath::zero,
        conf::LinearWorkspacePath::zero};

TEST_CASE("MI355X: linear projection reference, admission and lifetime") {
    Fixture f;
    RawStorageOracle oracle;
    conf::run_linear_conformance(f.devices(), kLinearDeclaration, &f.gate, &oracle);
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X: SDPA admission and BF16 attention on the matrix cores") {
    Fixture f;
    RawStorageOracle native_storage;
    const conf::SdpaNativeFailureSeam native_failure{
            [] { arm(seams::SubmissionFault::sdpa_launch); },
            [] { disarm(); },
            "rocm_detail::SubmissionFault::sdpa_launch",
            {}};
    const conf::SdpaConformanceConfig config{
            f.devices(), conf::kSdpaCurrentSupportedDataTypes, true, &f.gate, &native_storage, {},
            native_failure};
    conf::run_sdpa_conformance(config);
    CHECK_FALSE(f.gate.armed());
}

// ---- the composed suite a backend driver runs last ---------------------------------------------

TEST_CASE("MI355X: full shared suite with the RoPE contract") {
    Fixture f;
    RawStorageOracle oracle;
    const conf::RopeContractConformanceConfig rope_contract{
            f.devices(),
            conf::rope_reference::kRopeRocmExpectedSupported,
            &f.gate,
            conf::RopeNativeFailureSeam{
                    [] { arm(seams::SubmissionFault::event_record); },
                    [] { disarm(); },
                    "rocm_detail::SubmissionFault::event_record",
                    {}}};
    conf::run_backend_conformance(
            f.devices(), f.candidate->supported_data_types().subspan(0, 1), &f.gate, &oracle, true,
            true, &rope_contract, true);
    CHECK_FALSE(f.gate.armed());
}

// ---- what the reference's accelerator driver asserts through backend seams ----------------------
//
// test/rocm/test_rocm_conformance.cpp holds, beside the shared runners above, scenarios written
// against the reference ROCm backend's own fault seams (a failed launch, a failed event record, a
// failed status copy) and against owner addresses.  The same behaviours, asked of this backend
// through its own seams (mi355x_testing.hpp: one launch per operation, so the reference's "third
// plane launch" is `kernel_launch` here), with the reference's shared helpers for data and
// expected values.

namespace {

using Owner = std::unique_ptr<iom::Tensor>;

// Owners created now must not sit where the given (released) owners sat.
void expect_not_recycled(iom::Device& device, std::initializer_list<iom::TensorSpec> specs,
                         std::initializer_list<const void*> retired) {
    std::vector<Owner> fresh;
    for (const iom::TensorSpec& spec : specs) {
        fresh.push_back(device.create_tensor(spec));
    }
    for (const Owner& owner : fresh) {
        for (const void* address : retired) {
            CHECK_NE(static_cast<const void*>(owner->view().native_handle()), address);
        }
    }
}

// Raw tiled bytes of an owner, through the oracle above.
std::vector<std::byte> raw_storage(RawStorageOracle& oracle, const iom::TensorSpec& spec, const iom::TensorView& view) {
    oracle.set_owner_spec(spec);
    return oracle.observe(view);
}

}  // namespace

TEST_CASE("MI355X backend: a launch that fails after acceptance repeats its failure and the owners serve the next one") {
    const auto device = make_candidate();
    const iom::TensorSpec spec{iom::TensorShape{{2, 16, 16}}, iom::DataType::U8};
    auto lhs = device->create_tensor(spec);
    auto out = device->create_tensor(spec);
    std::vector<std::byte> pattern(spec.logical_nbytes());
    for (std::size_t i = 0; i < pattern.size(); ++i) {
        pattern[i] = static_cast<std::byte>((i * 5 + 1) & 0xff);
    }
    conf::copy_from_host(lhs->view(), pattern);
    auto queue = device->create_ops();

    arm(seams::SubmissionFault::kernel_launch);
    const iom::oid failed = queue->add(lhs->view(), lhs->view(), out->view());
    disarm();
    REQUIRE(iom::oid_is_token(failed));
    conf::expect_repeated_runtime_failure(*queue, failed);

    const iom::oid next = queue->add(lhs->view(), lhs->view(), out->view());
    REQUIRE(iom::oid_is_token(next));
    CHECK_EQ(conf::token_sequence(next), conf::token_sequence(failed) + 1);
    CHECK_NOTHROW(queue->wait(next));
    const std::vector<std::byte> doubled = conf::read_logical(out->view());
    for (std::size_t i = 0; i < doubled.size(); ++i) {
        CHECK_EQ(static_cast<unsigned>(doubled[i]), (static_cast<unsigned>(pattern[i]) * 2u) & 0xffu);
    }
}

TEST_CASE("MI355X backend: only accepted submissions take a sequence, and a failed one's operands are not recycled") {
    const auto device = make_candidate();
    const iom::TensorSpec spec{iom::TensorShape{{3, 16, 16}}, iom::DataType::U8};
    const iom::TensorSpec other{iom::TensorShape{{3, 16, 17}}, iom::DataType::U8};
    auto source = device->create_tensor(spec);
    auto destination = device->create_tensor(spec);
    auto misfit = device->create_tensor(other);
    const std::vector<std::byte> bytes(spec.logical_nbytes(), std::byte{0x3c});
    conf::copy_from_host(source->view(), bytes);
    conf::copy_from_host(destination->view(), bytes);
    auto queue = device->create_ops();

    // rejected by validation, then by a completion resource that cannot be had: no sequence
    CHECK_EQ(queue->copy(source->view(), misfit->view()), iom::to_oid(iom::OidError::InvalidArgument));
    const iom::oid first = queue->copy(source->view(), destination->view());
    CHECK_EQ(conf::token_sequence(first), 1u);
    CHECK_NOTHROW(queue->wait(first));
    arm(seams::SubmissionFault::event_create);
    CHECK_EQ(queue->copy(source->view(), destination->view()), iom::to_oid(iom::OidError::DeviceError));
    const iom::oid second = queue->copy(source->view(), destination->view());
    CHECK_EQ(conf::token_sequence(second), 2u);
    CHECK_NOTHROW(queue->wait(second));

    // accepted, then failed: the launch, and the record of the completion event
    arm(seams::SubmissionFault::kernel_launch);
    const iom::oid third = queue->copy(source->view(), destination->view());
    CHECK_EQ(conf::token_sequence(third), 3u);
    conf::expect_repeated_runtime_failure(*queue, third);
    arm(seams::SubmissionFault::event_record);
    const iom::oid fourth = queue->copy(source->view(), destination->view());
    CHECK_EQ(conf::token_sequence(fourth), 4u);
    conf::expect_repeated_runtime_failure(*queue, fourth);
    disarm();

    // a second device: the owners of a failed copy go away, their ranges do not come back
    {
        const auto second_device = make_candidate();
        auto a = second_device->create_tensor(spec);
        auto b = second_device->create_tensor(spec);
        auto doomed = second_device->create_ops();
        arm(seams::SubmissionFault::kernel_launch);
        const iom::oid failure = doomed->copy(a->view(), b->view());
        disarm();
        CHECK_EQ(conf::token_sequence(failure), 1u);
        conf::expect_repeated_runtime_failure(*doomed, failure);
        const void* was_a = a->view().native_handle();
        const void* was_b = b->view().native_handle();
        a.reset();
        b.reset();
        expect_not_recycled(*second_device, {spec, spec}, {was_a, was_b});
    }
}

TEST_CASE("MI355X backend: queue destruction drains pending copies around a failed one") {
    const auto device = make_candidate();
    const iom::TensorSpec spec{iom::TensorShape{{3, 16, 16}}, iom::DataType::U8};
    auto source = device->create_tensor(spec);
    auto destination = device->create_tensor(spec);
    const std::vector<std::byte> bytes(spec.logical_nbytes(), std::byte{0x5a});
    conf::copy_from_host(source->view(), bytes);
    conf::copy_from_host(destination->view(), bytes);
    {
        auto queue = device->create_ops();
        for (int i = 0; i < 32; ++i) {
            CHECK(iom::oid_is_token(queue->copy(source->view(), destination->view())));
        }
        arm(seams::SubmissionFault::kernel_launch);
        CHECK(iom::oid_is_token(queue->copy(source->view(), destination->view())));
        for (int i = 0; i < 32; ++i) {
            CHECK(iom::oid_is_token(queue->copy(source->view(), destination->view())));
        }
    }
    disarm();
    conf::require_logical_bytes(destination->view(), bytes, "destination after the drained queue");
}

TEST_CASE("MI355X backend: a source destroyed before the wait stays intact until both of its copies are done") {
    const iom::TensorSpec spec{iom::TensorShape{{8192, 4096}}, iom::DataType::F32};       // 128 MiB
    const std::vector<std::byte> expected = conf::encode_standard_tiled_storage(spec);
    const std::vector<std::byte> zeros(spec.tiled_storage_nbytes(), std::byte{0});
    const auto device = make_candidate();
    RawStorageOracle oracle;
    auto source = device->create_tensor(spec);
    auto first_destination = device->create_tensor(spec);
    auto second_destination = device->create_tensor(spec);
    oracle.set_owner_spec(spec);
    oracle.seed(source->view(), expected);
    oracle.seed(first_destination->view(), zeros);
    oracle.seed(second_destination->view(), zeros);
    auto queue = device->create_ops();
    const iom::oid first = queue->copy(source->view(), first_destination->view());
    const iom::oid second = queue->copy(source->view(), second_destination->view());
    source.reset();
    auto fresh = device->create_tensor(spec);       // zero-filled at creation, wherever it lands
    CHECK_NOTHROW(queue->wait(first));
    CHECK_NOTHROW(queue->wait(second));
    CHECK(raw_storage(oracle, spec, first_destination->view()) == expected);
    CHECK(raw_storage(oracle, spec, second_destination->view()) == expected);
}

TEST_CASE("MI355X backend: operands of work nobody waited for are quarantined once their queue is gone") {
    const iom::TensorSpec spec{iom::TensorShape{{4096, 2048}}, iom::DataType::F32};
    const auto device = make_candidate();
    auto source = device->create_tensor(spec);
    auto destination = device->create_tensor(spec);
    {
        auto queue = device->create_ops();
        CHECK(iom::oid_is_token(queue->copy(source->view(), destination->view())));
    }
    const void* was_source = source->view().native_handle();
    const void* was_destination = destination->view().native_handle();
    source.reset();
    destination.reset();
    expect_not_recycled(*device, {spec, spec}, {was_source, was_destination});
}

TEST_CASE("MI355X backend: cache append failures retire, a new queue appends correctly, pending operands are quarantined") {
    const auto device = make_candidate();
    struct Shape { std::vector<std::size_t> source, destination; std::size_t position; seams::SubmissionFault fault; };
    const Shape shapes[] = {
            {{1, 1, 1, 17}, {1, 1, 17, 17}, 1, seams::SubmissionFault::event_record},
            {{2, 1, 1, 33}, {2, 1, 33, 33}, 15, seams::SubmissionFault::kernel_launch}};
    std::uint64_t salt = 0x7c0;
    for (const Shape& shape : shapes) {
        const iom::TensorSpec source_spec{iom::TensorShape{shape.source}, iom::DataType::F32};
        const iom::TensorSpec destination_spec{iom::TensorShape{shape.destination}, iom::DataType::F32};
        auto source = device->create_tensor(source_spec);
        auto destination = device->create_tensor(destination_spec);
        const std::vector<std::byte> row = conf::encode_cache_append_logical(source_spec, ++salt);
        conf::copy_from_host(source->view(), row);
        conf::copy_from_host(destination->view(), conf::encode_logical(destination_spec, ++salt));
        auto queue = device->create_ops();
        arm(shape.fault);
        const iom::oid failed = queue->cache_append(source->view(), destination->view(), shape.position);
        disarm();
        REQUIRE(iom::oid_is_token(failed));
        conf::expect_repeated_runtime_failure(*queue, failed);

        auto other_destination = device->create_tensor(destination_spec);
        const std::vector<std::byte> before = conf::encode_logical(destination_spec, ++salt);
        conf::copy_from_host(other_destination->view(), before);
        auto other_queue = device->create_ops();
        const iom::oid appended = other_queue->cache_append(source->view(), other_destination->view(), shape.position);
        REQUIRE(iom::oid_is_token(appended));
        CHECK_NOTHROW(other_queue->wait(appended));
        CHECK_NOTHROW(other_queue->wait(appended));
        conf::require_logical_bytes(
                other_destination->view(),
                conf::cache_append_expected_logical(source_spec, destination_spec, shape.position, row, before),
                "append on a new queue after a retired failure");
    }
    // appends pending (one of them failed) when the queue goes: their operands do not come back
    {
        const iom::TensorSpec source_spec{iom::TensorShape{{3, 16, 16}}, iom::DataType::U8};
        const iom::TensorSpec destination_spec{iom::TensorShape{{3, 64, 16}}, iom::DataType::U8};
        auto source = device->create_tensor(source_spec);
        auto destination = device->create_tensor(destination_spec);
        conf::copy_from_host(source->view(), conf::encode_cache_append_logical(source_spec, ++salt));
        conf::copy_from_host(destination->view(), conf::encode_logical(destination_spec, ++salt));
        const void* was_source = source->view().native_handle();
        const void* was_destination = destination->view().native_handle();
        {
            auto queue = device->create_ops();
            for (int i = 0; i < 4; ++i) {
                CHECK(iom::oid_is_token(queue->cache_append(source->view(), destination->view(), 1)));
            }
            arm(seams::SubmissionFault::kernel_launch);
            CHECK(iom::oid_is_token(queue->cache_append(source->view(), destination->view(), 1)));
        }
        disarm();
        source.reset();
        destination.reset();
        expect_not_recycled(*device, {source_spec, destination_spec}, {was_source, was_destination});
    }
    // a large source destroyed right after submission is still what gets appended
    {
        const iom::TensorSpec source_spec{iom::TensorShape{{32, 1, 8192, 128}}, iom::DataType::U8};
        const iom::TensorSpec destination_spec{iom::TensorShape{{32, 1, 16384, 128}}, iom::DataType::U8};
        auto source = device->create_tensor(source_spec);
        auto destination = device->create_tensor(destination_spec);
        const std::vector<std::byte> rows = conf::encode_cache_append_logical(source_spec, ++salt);
        const std::vector<std::byte> before = conf::encode_logical(destination_spec, ++salt);
        conf::copy_from_host(source->view(), rows);
        conf::copy_from_host(destination->view(), before);
        auto queue = device->create_ops();
        const iom::oid token = queue->cache_append(source->view(), destination->view(), 17);
        REQUIRE(iom::oid_is_token(token));
        source.reset();
        auto intruder = device->create_tensor(source_spec);
        conf::copy_from_host(intruder->view(), conf::encode_cache_append_logical(source_spec, ++salt));
        CHECK_NOTHROW(queue->wait(token));
        conf::require_logical_bytes(
                destination->view(),
                conf::cache_append_expected_logical(source_spec, destination_spec, 17, rows, before),
                "append whose source owner went away before the wait");
    }
}

TEST_CASE("MI355X backend: an embedding whose status word cannot be fetched retires as failed and the queue goes on") {
    const auto device = make_candidate();
    const iom::TensorSpec table_spec{iom::TensorShape{{4, 8}}, iom::DataType::U8};
    const iom::TensorSpec index_spec{iom::TensorShape{{1, 8}}, iom::DataType::U32};
    const iom::TensorSpec output_spec{iom::TensorShape{{8, 8}}, iom::DataType::U8};
    auto table = device->create_tensor(table_spec);
    auto indices = device->create_tensor(index_spec);
    auto output = device->create_tensor(output_spec);
    conf::copy_from_host(table->view(), std::vector<std::byte>(table_spec.logical_nbytes()));
    conf::copy_from_host(indices->view(), std::vector<std::byte>(index_spec.logical_nbytes()));
    auto workspace = device->create_workspace(32);
    auto queue = device->create_ops();
    for (const seams::SubmissionFault fault :
         {seams::SubmissionFault::embedding_status_copy, seams::SubmissionFault::kernel_launch}) {
        arm(fault);
        const iom::oid failed = queue->embedding(table->view(), indices->view(), output->view(), workspace->view());
        disarm();
        REQUIRE(iom::oid_is_token(failed));
        conf::expect_repeated_runtime_failure(*queue, failed);
        const iom::oid next = queue->embedding(table->view(), indices->view(), output->view(), workspace->view());
        REQUIRE(iom::oid_is_token(next));
        CHECK_NOTHROW(queue->wait(next));
    }
}

TEST_CASE("MI355X backend: SiLU launch evidence, accepted failure, recovery, and quarantine after an unrecorded completion") {
    const auto device = make_candidate();
    {
        const conf::SiluReferenceCase fixture = conf::silu_make_pattern_case(
                conf::SiluReferenceCaseKind::ordinary, iom::DataType::F32, {2}, 2, 17, "mi355x-failure/F32");
        const iom::TensorSpec spec = conf::silu_case_spec(fixture);
        auto input = device->create_tensor(spec);
        auto output = device->create_tensor(spec);
        const std::vector<std::byte> input_bytes = conf::silu_pack_bits(iom::DataType::F32, fixture.input_bits);
        conf::copy_from_host(input->view(), input_bytes);
        conf::copy_from_host(output->view(), std::vector<std::byte>(spec.logical_nbytes(), conf::kReadbackSentinel));
        const std::vector<conf::SiluReferenceValue> expected = conf::silu_evaluate(fixture);
        auto queue = device->create_ops();
        const std::size_t launches = seams::silu_launch_count_for_testing.load();
        const iom::oid healthy = queue->silu(input->view(), output->view());
        REQUIRE(iom::oid_is_token(healthy));
        CHECK_NOTHROW(queue->wait(healthy));
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), launches + 1);
        // the fault is consumed before the launch: accepted, failed, and no kernel ran
        arm(seams::SubmissionFault::silu_launch);
        const iom::oid failed = queue->silu(input->view(), output->view());
        disarm();
        REQUIRE(iom::oid_is_token(failed));
        CHECK_EQ(conf::token_sequence(failed), conf::token_sequence(healthy) + 1);
        conf::expect_repeated_runtime_failure(*queue, failed);
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), launches + 1);
        const iom::oid again = queue->silu(input->view(), output->view());
        REQUIRE(iom::oid_is_token(again));
        CHECK_EQ(conf::token_sequence(again), conf::token_sequence(failed) + 1);
        CHECK_NOTHROW(queue->wait(again));
        CHECK_NOTHROW(queue->wait(again));
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), launches + 2);
        const std::string mismatch = conf::silu_compare(
                iom::DataType::F32, conf::read_logical(output->view()), expected, "activation after the failure");
        CHECK_MESSAGE(mismatch.empty(), mismatch);
        conf::require_logical_bytes(input->view(), input_bytes, "input after the failure");
    }
    {
        // the completion event cannot be recorded: the operands stay out of the arena, and fresh
        // operands on a fresh queue give the reference activation
        const conf::SiluReferenceCase fixture = conf::silu_make_pattern_case(
                conf::SiluReferenceCaseKind::boundary_sizes, iom::DataType::BF16, {2}, 17, 17, "mi355x-unrecorded/BF16");
        const iom::TensorSpec spec = conf::silu_case_spec(fixture);
        const std::vector<std::byte> input_bytes = conf::silu_pack_bits(iom::DataType::BF16, fixture.input_bits);
        const std::vector<conf::SiluReferenceValue> expected = conf::silu_evaluate(fixture);
        auto input = device->create_tensor(spec);
        auto output = device->create_tensor(spec);
        conf::copy_from_host(input->view(), input_bytes);
        const void* was_input = input->view().native_handle();
        const void* was_output = output->view().native_handle();
        {
            auto queue = device->create_ops();
            arm(seams::SubmissionFault::event_record);
            const iom::oid failed = queue->silu(input->view(), output->view());
            disarm();
            REQUIRE(iom::oid_is_token(failed));
            conf::expect_repeated_runtime_failure(*queue, failed);
        }
        input.reset();
        output.reset();
        auto fresh_input = device->create_tensor(spec);
        auto fresh_output = device->create_tensor(spec);
        for (const void* retired : {was_input, was_output}) {
            CHECK_NE(static_cast<const void*>(fresh_input->view().native_handle()), retired);
            CHECK_NE(static_cast<const void*>(fresh_output->view().native_handle()), retired);
        }
        conf::copy_from_host(fresh_input->view(), input_bytes);
        conf::copy_from_host(fresh_output->view(),
                             std::vector<std::byte>(spec.logical_nbytes(), conf::kReadbackSentinel));
        auto queue = device->create_ops();
        const iom::oid token = queue->silu(fresh_input->view(), fresh_output->view());
        REQUIRE(iom::oid_is_token(token));
        CHECK_NOTHROW(queue->wait(token));
        const std::string mismatch = conf::silu_compare(
                iom::DataType::BF16, conf::read_logical(fresh_output->view()), expected, "activation on fresh operands");
        CHECK_MESSAGE(mismatch.empty(), mismatch);
    }
}

TEST_CASE("MI355X backend: SiLU submitted through views that die before the wait, input owner destroyed first") {
    // the reference driver's scenario (test/rocm/test_rocm_conformance.cpp:1494-1572): both
    // descriptors handed to silu() are temporaries of the submitting call, the input owner goes
    // away before the token is observed, and the poisoned padding of the output owner survives
    const auto device = make_candidate();
    const iom::TensorSpec owner_spec = conf::silu_make_spec({3, 4, 2, 17}, iom::DataType::F16);
    const conf::SiluReferenceCase fixture = conf::silu_make_pattern_case(
            conf::SiluReferenceCaseKind::ordinary, iom::DataType::F16, {2, 2}, 2, 17, "mi355x-temporary/F16");
    const iom::TensorSpec logical_spec = conf::silu_case_spec(fixture);
    const std::vector<std::byte> input_logical = conf::silu_pack_bits(iom::DataType::F16, fixture.input_bits);
    const std::vector<conf::SiluReferenceValue> expected = conf::silu_evaluate(fixture);
    const std::vector<std::byte> poison(logical_spec.logical_nbytes(), conf::kReadbackSentinel);
    auto input_owner = device->create_tensor(owner_spec);
    auto output_owner = device->create_tensor(owner_spec);
    RawStorageOracle storage;
    {
        iom::TensorView input_view = conf::silu_transformed_view(*input_owner);
        iom::TensorView output_view = conf::silu_transformed_view(*output_owner);
        REQUIRE(input_view.spec() == logical_spec);
        REQUIRE(output_view.spec() == logical_spec);
        storage.set_owner_spec(owner_spec);
        storage.seed(input_view, conf::silu_storage_image(owner_spec, input_view, input_logical, std::byte{0x5A}));
        storage.set_owner_spec(owner_spec);
        storage.seed(output_view, conf::silu_storage_image(owner_spec, output_view, poison, std::byte{0xA5}));
        auto queue = device->create_ops();
        const auto submit = [&queue](iom::Tensor& input, iom::Tensor& output) {
            const iom::TensorView in = conf::silu_transformed_view(input);
            iom::TensorView out = conf::silu_transformed_view(output);
            return queue->silu(in, out);
        };
        const iom::oid token = submit(*input_owner, *output_owner);
        REQUIRE(iom::oid_is_token(token));
        input_owner.reset();
        CHECK_NOTHROW(queue->wait(token));
        CHECK_NOTHROW(queue->wait(token));
        const std::vector<std::byte> activated = conf::read_logical(output_view);
        const std::string mismatch = conf::silu_compare(
                iom::DataType::F16, activated, expected, "activation through temporary views");
        CHECK_MESSAGE(mismatch.empty(), mismatch);
        std::vector<std::byte> want(owner_spec.tiled_storage_nbytes(), std::byte{0xA5});
        conf::apply_standard_tiled_view(output_view, owner_spec, activated, want);
        storage.set_owner_spec(owner_spec);
        CHECK(storage.observe(output_view) == want);
    }
    output_owner.reset();
}

TEST_CASE("MI355X backend: one SiLU kernel per accepted request of every floating leaf, none for a rejected one, negative subnormal tails kept") {
    // test/rocm/test_rocm_conformance.cpp:1578-1676 against this backend's launch counter
    const auto device = make_candidate();
    auto queue = device->create_ops();
    for (const iom::DataType type : conf::kSiluRocmExpectedSupported) {
        CAPTURE(static_cast<int>(type));
        const iom::TensorSpec spec = conf::silu_make_spec({2, 17, 17}, type);
        auto input = device->create_tensor(spec);
        auto output = device->create_tensor(spec);
        const std::size_t before = seams::silu_launch_count_for_testing.load();
        const iom::oid token = queue->silu(input->view(), output->view());
        REQUIRE(iom::oid_is_token(token));
        CHECK_NOTHROW(queue->wait(token));
        CHECK_NOTHROW(queue->wait(token));
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), before + 1);
    }
    {
        const iom::TensorSpec spec = conf::silu_make_spec({2, 17, 17}, iom::DataType::F32);
        const iom::TensorSpec other = conf::silu_make_spec({2, 17, 18}, iom::DataType::F32);
        auto input = device->create_tensor(spec);
        auto output = device->create_tensor(other);
        const std::size_t before = seams::silu_launch_count_for_testing.load();
        CHECK_EQ(queue->silu(input->view(), output->view()), iom::to_oid(iom::OidError::InvalidArgument));
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), before);
        CHECK_EQ(queue->silu(input->view(), input->view()), iom::to_oid(iom::OidError::InvalidArgument));
        CHECK_EQ(seams::silu_launch_count_for_testing.load(), before);
    }
    for (const iom::DataType type : {iom::DataType::F32, iom::DataType::F64}) {
        CAPTURE(static_cast<int>(type));
        const conf::SiluReferenceCase tails = conf::silu_make_tail_case(type);
        const iom::TensorSpec spec = conf::silu_case_spec(tails);
        auto input = device->create_tensor(spec);
        auto output = device->create_tensor(spec);
        conf::copy_from_host(input->view(), conf::silu_pack_bits(type, tails.input_bits));
        conf::copy_from_host(output->view(), std::vector<std::byte>(spec.logical_nbytes(), conf::kReadbackSentinel));
        const iom::oid token = queue->silu(input->view(), output->view());
        REQUIRE(iom::oid_is_token(token));
        CHECK_NOTHROW(queue->wait(token));
        const std::vector<std::byte> observed = conf::read_logical(output->view());
        const std::vector<conf::SiluReferenceValue> expected = conf::silu_evaluate(tails);
        const std::uint64_t tail_input =
                conf::silu_oracle::value_bits(type, type == iom::DataType::F64 ? -746.0 : -104.0);
        std::size_t seen = 0;
        for (std::size_t i = 0; i < expected.size(); ++i) {
            if (tails.input_bits[i] != tail_input) continue;
            ++seen;
            const std::uint64_t bits = conf::silu_read_bits(observed, type, i);
            CHECK_EQ(bits, expected[i].bits);
            // classified in the leaf's own domain: a binary32 subnormal widened to binary64 is normal
            bool negative_subnormal = false;
            if (type == iom::DataType::F64) {
                const double v = conf::silu_oracle::decode_f64(bits);
                negative_subnormal = std::fpclassify(v) == FP_SUBNORMAL && std::signbit(v);
            } else {
                const float v = conf::silu_oracle::decode_f32(type, bits);
                negative_subnormal = std::fpclassify(v) == FP_SUBNORMAL && std::signbit(v);
            }
            CHECK_MESSAGE(negative_subnormal, "the tail must stay a nonzero negative subnormal");
        }
        CHECK(seen > 0);
    }
}

TEST_CASE("MI355X backend: TinyLlama-shaped attention, prefill of 17 rows and the decode step that follows it") {
    Fixture f;
    RawStorageOracle native_storage;
    const conf::SdpaConformanceConfig config{
            f.devices(), conf::kSdpaCurrentSupportedDataTypes, true, &f.gate, &native_storage, {}, {}};
    const conf::SdpaReferenceCase prefill = conf::sdpa_oracle::make_exact_capacity_case(iom::DataType::BF16);
    const conf::SdpaReferenceCase decode = conf::sdpa_incremental_slice(prefill, prefill.rows - 1);
    REQUIRE_EQ(prefill.rows, std::size_t{17});
    REQUIRE_EQ(decode.rows, std::size_t{1});
    (void)conf::sdpa_detail::run_reference_case(config, prefill, "prefill of 17 rows");
    (void)conf::sdpa_detail::run_reference_case(config, decode, "decode step");
    CHECK_FALSE(f.gate.armed());
}

TEST_CASE("MI355X backend: workspaces are ranges of the one arena, and requirement queries are pure") {
    const std::size_t allocations = seams::device_allocation_count_for_testing.load();
    const auto device = iom::make_rocm_device(0, iom::DeviceMemoryConfig{1u * 1024 * 1024});
    CHECK_EQ(seams::device_allocation_count_for_testing.load(), allocations + 1);     // the arena itself
    auto empty = device->create_workspace(0);
    REQUIRE(empty != nullptr);
    CHECK(empty->empty());
    CHECK_EQ(empty->byte_size(), std::size_t{0});
    CHECK(empty->view().owner_identity() == empty.get());
    CHECK(&empty->view().device() == device.get());
    auto workspace = device->create_workspace(4096);
    REQUIRE(workspace != nullptr);
    const iom::RawWorkspaceView view = workspace->view();
    CHECK_EQ(view.byte_size(), std::size_t{4096});
    CHECK(view.owner_identity() == workspace.get());
    CHECK_NOTHROW((void)iom::detail::WorkspaceValidation::validated(*device, view, 4096, 32, {}));
    auto another = device->create_workspace(256);
    REQUIRE(another != nullptr);
    CHECK(workspace->view() == view);                                                 // stable
    CHECK_THROWS_AS((void)device->create_workspace(2u * 1024 * 1024), std::bad_alloc);
    another.reset();
    auto reused = device->create_workspace(256);
    REQUIRE(reused != nullptr);
    CHECK_EQ(reused->byte_size(), std::size_t{256});
    CHECK_EQ(seams::device_allocation_count_for_testing.load(), allocations + 1);     // nothing since

    // queries: no workspace for the binary operations, the staged logical bytes for host transfers
    Fixture f;
    const iom::TensorSpec spec{iom::TensorShape{{2, 3, 17, 33}}, iom::DataType::F32};
    auto lhs = f.candidate->create_tensor(spec);
    auto rhs = f.candidate->create_tensor(spec);
    auto out = f.candidate->create_tensor(spec);
    auto queue = f.candidate->create_ops();
    const iom::WorkspaceRequirements none{0, 1};
    for (int repeat = 0; repeat < 2; ++repeat) {
        CHECK(queue->add_workspace_requirements(lhs->view(), rhs->view(), out->view()) == none);
        CHECK(queue->mul_workspace_requirements(lhs->view(), rhs->view(), out->view()) == none);
        CHECK(queue->sub_workspace_requirements(lhs->view(), rhs->view(), out->view()) == none);
        CHECK(queue->div_workspace_requirements(lhs->view(), rhs->view(), out->view()) == none);
    }
    const iom::WorkspaceRequirements staged{iom::gpu_algorithm::compute_staging_size(spec.logical_nbytes()), 32};
    CHECK(lhs->view().copy_from_host_workspace_requirements() == staged);
    CHECK(lhs->view().copy_to_host_workspace_requirements() == staged);
    auto foreign_tensor = f.reference->create_tensor(spec);
    CHECK_THROWS_AS((void)queue->add_workspace_requirements(foreign_tensor->view(), rhs->view(), out->view()),
                    std::invalid_argument);
}

int main(int argc, char** argv) {
    int devices = 0;
    if (iomx_device_count(&devices) != IOMX_OK || devices < 1) {
        std::fprintf(stderr, "mi355x_conformance: no HIP device\n");
        return 3;
    }
    doctest::Context context(argc, argv);
    return context.run();
}
