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

int main(int argc, char** argv) {
    int devices = 0;
    if (iomx_device_count(&devices) != IOMX_OK || devices < 1) {
        std::fprintf(stderr, "mi355x_conformance: no HIP device\n");
        return 3;
    }
    doctest::Context context(argc, argv);
    return context.run();
}
