// CPU check of the packing helpers and the element arithmetic of iomx_leaves.hip (plain C++
// functions usable from host code) against the oracle: exhaustive over every operand pair of
// the leaves of at most 8 bits, sampled for the wider ones.  Built and run by
// tests/test_leaves_host_check.py; exits nonzero on any mismatch.
#include "iomx_leaves.hip"
#include "iom_oracle.h"
#include <cstdio>
#include <cstdlib>
#include <vector>
namespace iomx { void record_launch(const char*, uint32_t, uint32_t, uint64_t) {} }
using namespace iomx;

static uint64_t rng_state = 88172645463325252ull;
static uint64_t rnd() { rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17; return rng_state; }

template <int DT> long check_binary_exhaustive() {
    constexpr int BITS = bits_of(DT);
    long bad = 0;
    const uint64_t n = 1ull << BITS;
    for (uint64_t a = 0; a < n; ++a) for (uint64_t b = 0; b < n; ++b) {
        const uint64_t r0 = leaf_binary<DT, IOMX_OP_ADD>(a, b), r1 = leaf_binary<DT, IOMX_OP_MUL>(a, b), r2 = leaf_binary<DT, IOMX_OP_SUB>(a, b);
        const uint64_t w0 = iomo_scalar_binary(0, DT, a, b), w1 = iomo_scalar_binary(1, DT, a, b), w2 = iomo_scalar_binary(2, DT, a, b);
        if (r0 != w0 || r1 != w1 || r2 != w2) { if (bad < 5) printf("dt %d a %llx b %llx: %llx %llx %llx want %llx %llx %llx\n", DT, (unsigned long long)a, (unsigned long long)b, (unsigned long long)r0,(unsigned long long)r1,(unsigned long long)r2,(unsigned long long)w0,(unsigned long long)w1,(unsigned long long)w2); ++bad; }
    }
    return bad;
}
template <int DT> long check_binary_random(long count, bool codec) {
    constexpr int BITS = bits_of(DT);
    long bad = 0;
    const uint64_t mask = BITS == 64 ? ~0ull : (1ull << BITS) - 1;
    for (long i = 0; i < count; ++i) {
        uint64_t a = rnd() & mask, b = rnd() & mask;
        if (i % 7 == 0) b = a ^ (rnd() & 3);           // near-cancellation
        if (i % 11 == 0) b = (a & ~(mask >> 1)) ^ (rnd() & mask >> 1) ;
        for (int op = 0; op < 3; ++op) {
            const uint64_t r = op == 0 ? leaf_binary<DT, 0>(a, b) : op == 1 ? leaf_binary<DT, 1>(a, b) : leaf_binary<DT, 2>(a, b);
            const uint64_t w = codec ? iomo_scalar_binary(op, DT, a, b) : iomo_scalar_binary_ieee(op, DT, a, b);
            if (r != w) { if (bad < 5) printf("dt %d op %d a %llx b %llx: %llx want %llx\n", DT, op, (unsigned long long)a, (unsigned long long)b, (unsigned long long)r, (unsigned long long)w); ++bad; }
        }
    }
    return bad;
}
template <int DT> long check_silu(bool exhaustive) {
    constexpr int BITS = bits_of(DT);
    long bad = 0, off = 0;
    const uint64_t n = exhaustive ? (1ull << BITS) : 200000;
    const uint64_t mask = BITS == 64 ? ~0ull : (1ull << BITS) - 1;
    for (uint64_t i = 0; i < n; ++i) {
        const uint64_t a = exhaustive ? i : (rnd() & mask);
        const uint64_t r = leaf_silu<DT>(a), w = iomo_scalar_silu(DT, a);
        if (r != w) { ++off; const long long d = (long long)r - (long long)w; if (d > 2 || d < -2) { if (bad < 5) printf("silu dt %d a %llx: %llx want %llx\n", DT, (unsigned long long)a, (unsigned long long)r, (unsigned long long)w); ++bad; } }
    }
    printf("silu dt %d: %ld differ by <=2 (host libm on both sides), %ld worse\n", DT, off, bad);
    return bad;
}
template <int BITS> long check_packing() {
    constexpr int K = BITS / 2;
    long bad = 0;
    for (int trial = 0; trial < 2000; ++trial) {
        alignas(16) uint32_t mem[K + 4];
        uint64_t vals[16];
        const uint64_t mask = BITS == 64 ? ~0ull : (1ull << BITS) - 1;
        uint32_t w[K] = {};
        for (int i = 0; i < 16; ++i) { vals[i] = rnd() & mask; put<BITS>(w, i, vals[i]); }
        for (int i = 0; i < 16; ++i) if (get<BITS>(w, i) != vals[i]) ++bad;
        // bit-serial view of w must match
        for (int i = 0; i < 16; ++i) for (int k = 0; k < BITS; ++k) {
            const int bit = i * BITS + k;
            if (((w[bit >> 5] >> (bit & 31)) & 1) != ((vals[i] >> k) & 1)) ++bad;
        }
        for (uint32_t ncols = 1; ncols <= 16; ++ncols) {
            uint32_t before[K + 4];
            for (int j = 0; j < K + 4; ++j) before[j] = mem[j] = (uint32_t)rnd();
            store_row<BITS>(reinterpret_cast<uint8_t*>(mem), w, ncols);
            for (int bit = 0; bit < (K + 4) * 32; ++bit) {
                const uint32_t got = (mem[bit >> 5] >> (bit & 31)) & 1;
                const uint32_t want = bit < (int)ncols * BITS ? (w[bit >> 5] >> (bit & 31)) & 1 : (before[bit >> 5] >> (bit & 31)) & 1;
                if (got != want) ++bad;
            }
            uint32_t back[K];
            load_row<BITS>(reinterpret_cast<const uint8_t*>(mem), back);
            for (uint32_t i = 0; i < ncols; ++i) if (get<BITS>(back, i) != vals[i]) ++bad;
        }
        // read_bits at arbitrary element-aligned offsets of a stream
        uint32_t stream[64];
        for (auto& x : stream) x = (uint32_t)rnd();
        for (int e = 0; e * BITS + BITS <= 62 * 32; e += 1 + (int)(rnd() % 5)) {
            uint64_t want = 0;
            for (int k = 0; k < BITS; ++k) { const int bit = e * BITS + k; want |= (uint64_t)((stream[bit >> 5] >> (bit & 31)) & 1) << k; }
            if (read_bits<BITS>(stream, (uint64_t)e * BITS) != want) ++bad;
        }
    }
    return bad;
}
int main() {
    long bad = 0;
    bad += check_packing<2>() + check_packing<4>() + check_packing<6>() + check_packing<8>() + check_packing<16>() + check_packing<32>() + check_packing<64>();
    printf("packing mismatches so far: %ld\n", bad);
    bad += check_binary_exhaustive<DT_I2>() + check_binary_exhaustive<DT_I4>() + check_binary_exhaustive<DT_I8>();
    bad += check_binary_exhaustive<DT_F4_E2M1>() + check_binary_exhaustive<DT_F6_E2M3>() + check_binary_exhaustive<DT_F6_E3M2>();
    bad += check_binary_exhaustive<DT_F8_E4M3FN>() + check_binary_exhaustive<DT_F8_E5M2>();
    printf("after exhaustive narrow leaves: %ld\n", bad);
    bad += check_binary_random<DT_F16>(3000000, true) + check_binary_random<DT_I16>(100000, true) + check_binary_random<DT_I64>(100000, true);
    bad += check_binary_random<DT_F64>(3000000, false);
    printf("after F16/I16/I64/F64: %ld\n", bad);
    bad += check_silu<DT_F4_E2M1>(true) + check_silu<DT_F6_E2M3>(true) + check_silu<DT_F6_E3M2>(true) + check_silu<DT_F8_E4M3FN>(true)
         + check_silu<DT_F8_E5M2>(true) + check_silu<DT_F16>(true) + check_silu<DT_F64>(false);
    printf("TOTAL mismatches: %ld\n", bad);
    return bad != 0;
}
