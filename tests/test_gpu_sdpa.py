"""GPU parity of causal grouped-query attention, through the C ABI.

Checked against the reference's fixed fixtures and their expected values
(tests/golden/sdpa_reference_cases.json, acceptance rule of
test/backend/backend_conformance_sdpa_reference.hpp:1232-1259: same value class, and for
finite values at most two BF16 steps or 2^-10 absolute) and against the CPU oracle
(the reference CPU backend's arithmetic) on seeded shapes with the same rule.
"""
import numpy as np
import pytest

import datagen
import iomo
from iom_amd import iomx
from iomo import DT_BF16, DT_F32
from test_oracle_sdpa import CASES, all_match, matches, random_case, shapes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def device_operands(case, fill=0x5A):
    qd, kd, od = shapes(case)
    t = [iomx.DeviceTensor(DT_BF16, d, fill=fill) for d in (qd, kd, kd, od)]
    t[0].view().from_host(np.array(case["q"], np.uint16).reshape(qd))
    t[1].view().from_host(np.array(case["k"], np.uint16).reshape(kd))
    t[2].view().from_host(np.array(case["v"], np.uint16).reshape(kd))
    return t


def run(case, path, fill=0x5A, expect_kernel=None):
    q, k, v, o = device_operands(case, fill)
    before = o.raw().copy()
    ws = None
    if path in (0, 2):
        rc, nbytes, align = iomx.sdpa_workspace(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"])
        assert rc == 0 and align in (1, 256)
        ws = iomx.Buffer(nbytes) if nbytes else None
        if ws:
            ws.fill(0xEE)
    rc = iomx.sdpa(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"], ws, path)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    iomx.synchronize()
    if expect_kernel:
        assert iomx.last_launch().kernel.decode() == expect_kernel
    got = o.view().to_host()
    # nothing outside the logical output is written
    mask = iomo.tile_plane(np.ones(o.dims, np.uint16)) == 0
    assert np.array_equal(o.raw()[mask], before[mask])
    for t in (q, k, v, o):
        t.free()
    if ws:
        ws.free()
    return got


def oracle(case, fill=0x5A):
    from test_oracle_sdpa import host_operands
    q, k, v, o = host_operands(case, fill)
    assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"]) == 0
    return o.view().to_logical()


def close_to_oracle(got, want):
    got, want = got.reshape(-1), want.reshape(-1)
    from test_oracle_sdpa import bf16_class
    return [i for i, (g, w) in enumerate(zip(got, want)) if not matches(int(g), int(w), bf16_class(int(w)))]


@pytest.mark.parametrize("path,kernel", [(0, "sdpa_mfma"), (1, "sdpa_rows")], ids=["matrix_cores", "reference_order"])
@pytest.mark.parametrize("index", range(len(CASES)), ids=[c["label"].replace(" ", "_") for c in CASES])
def test_reference_fixtures(index, path, kernel):
    case = CASES[index]
    if path == 0 and (case["Hq"] // case["Hkv"]) * case["R"] <= 16:
        kernel = "sdpa_decode"        # all rows of a KV head's query heads fit one tile
    for fill in (0x5A, 0xFF):          # 0xFF: NaN patterns in tile padding
        got = run(case, path, fill, kernel)
        assert all_match(got, case) == [], case["label"]


SEEDED = [((), 2, 1, 5, 8, 12, 3, 9), ((2,), 4, 2, 17, 16, 40, 20, 37), ((2, 2), 4, 1, 3, 33, 20, 0, 2),
          ((), 8, 2, 1, 64, 70, 69, 70), ((3,), 2, 2, 16, 5, 16, 0, 16), ((2,), 8, 2, 40, 64, 100, 50, 90),
          ((), 4, 4, 33, 128, 64, 10, 43), ((), 2, 1, 70, 48, 200, 100, 170), ((), 8, 2, 33, 128, 64, 10, 43),
          ((2,), 4, 4, 70, 64, 100, 20, 90), ((), 6, 3, 100, 128, 120, 10, 110)]


def float64_attention(case):
    """Attention in float64 on the flushed operands, and per output the budget of the BF16
    probability: every P is rounded once to BF16 (2^-9 relative) and a score that differs in
    its last binary32 bits can move it one more step, so |error| <= 2^-8 * sum_t P|V|, plus the
    final BF16 rounding."""
    lead, Hq, Hkv, R, D, C, a, L = (case[k] for k in ("leading", "Hq", "Hkv", "R", "D", "C", "a", "L"))
    n = int(np.prod(lead)) if lead else 1

    def values(name, shape):
        bits = np.array(case[name], np.uint16).reshape(shape).copy()
        bits[(bits & 0x7F80) == 0] &= 0x8000
        return datagen.bf16_to_f32(bits.reshape(-1)).astype(np.float64).reshape(shape)
    q, k, v = values("q", (n, Hq, R, D)), values("k", (n, Hkv, C, D)), values("v", (n, Hkv, C, D))
    out = np.zeros((n, R, Hq * D))
    budget = np.zeros((n, R, Hq * D))
    for b in range(n):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            s = q[b, h] @ k[b, g, :L].T / np.sqrt(np.float32(D)).astype(np.float64)
            t = np.arange(L)[None, :]
            s = np.where(t <= a + np.arange(R)[:, None], s, -np.inf)
            e = np.exp(s - s.max(axis=1, keepdims=True))
            pr = e / e.sum(axis=1, keepdims=True)
            out[b, :, h * D:(h + 1) * D] = pr @ v[b, g, :L]
            budget[b, :, h * D:(h + 1) * D] = 2.0 ** -8 * (pr @ np.abs(v[b, g, :L]))
    return out, budget + 2.0 ** -8 * np.abs(out) + 2.0 ** -126


# seeded shapes whose matrix-core result has outputs outside the fixture rule, and how many
FIXTURE_RULE_CAP = {((2,), 8, 2, 40, 64, 100, 50, 90): 4}


@pytest.mark.parametrize("path", [0, 1, 2], ids=["matrix_cores", "reference_order", "two_tiles_a_wave"])
@pytest.mark.parametrize("spec", SEEDED, ids=[str(i) for i in range(len(SEEDED))])
def test_seeded_shapes_against_the_oracle(spec, path):
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(41 + R, lead, Hq, Hkv, R, D, C, a, L)
    kk = np.array(case["k"], np.uint16)
    kk[1], kk[2] = 0x0040, 0x8001         # subnormal operands: flushed
    case["k"] = kk.tolist()
    got = run(case, path, fill=0xFF)
    want = oracle(case)
    exact = int(np.sum(got.reshape(-1) == want.reshape(-1)))
    outside = close_to_oracle(got, want)
    print(spec, "path", path, "bit-equal to the oracle:", exact, "of", got.size,
          "outside the fixture rule:", len(outside), flush=True)
    ref64, budget = float64_attention(case)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)
    # the oracle itself sits inside the same budget, so the budget is not a loose one
    w = datagen.bf16_to_f32(want.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(w - ref64) <= budget)
    assert np.all(np.abs(g - w) <= 2 * budget)                 # hence within twice the budget of each other
    if path == 1:
        assert outside == [] and exact >= 0.98 * got.size     # same order of operations; only expf may differ
    else:
        # The reference's own acceptance rule for a native kernel -- two BF16 steps or 2^-10
        # (docs/BACKEND_CONTRACT/scaled-dot-product-attention.md:282-287) -- holds on every element of
        # every seeded shape but one, where 4 of 40960 outputs that cancel to near zero miss it (the
        # rule is not a bound under cancellation; the float64 budget above is, on every element).
        # That count is a cap: a kernel change that worsens it fails here.
        assert len(outside) <= FIXTURE_RULE_CAP.get(spec, 0), (spec, len(outside))


PAIRS = [((2,), 8, 2, 33, 64, 60, 20, 53), ((), 8, 2, 100, 128, 128, 0, 100), ((3,), 4, 1, 64, 64, 64, 0, 64),
         ((), 16, 4, 75, 128, 300, 200, 275), ((2,), 8, 2, 16, 64, 40, 3, 19), ((), 8, 2, 130, 64, 200, 50, 180)]


@pytest.mark.parametrize("spec", PAIRS, ids=[str(i) for i in range(len(PAIRS))])
def test_two_row_tiles_a_wave_equal_the_one_tile_kernel(spec):
    """The kernel that gives a wave two neighbouring row tiles (path 2; path 0 picks it from 1024 rows
    on) forms every row with the arithmetic of the one-tile kernel in the same order, so the outputs
    are the same bits: odd and even numbers of row tiles, a ragged last tile, rows that start behind
    a cached prefix, several planes."""
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(71, lead, Hq, Hkv, R, D, C, a, L)
    two = run(case, 2, fill=0xFF, expect_kernel="sdpa_mfma_pair")
    one = run(case, 0, fill=0xFF, expect_kernel="sdpa_mfma")
    if (L + 31) // 32 < 8:
        assert np.array_equal(two, one)
    else:
        # (a long prefix on few rows: path 0 shares the token groups out over the waves of a workgroup,
        # another order of additions)
        assert np.mean(two == one) > 0.99
    assert close_to_oracle(two, oracle(case)) == []


@pytest.mark.parametrize("D", [64, 128])
def test_a_prefill_of_1024_rows_takes_two_tiles_a_wave_by_itself(D):
    """From 1024 rows on (and enough row tiles, heads and planes to fill the chip without sharing a
    head's tokens among waves) path 0 itself gives a wave two row tiles."""
    n, Hq, Hkv, R = 4, 32, 8, 1024
    case = random_case(79, (n,), Hq, Hkv, R, D, R, 0, R)
    got = run(case, 0, expect_kernel="sdpa_mfma_pair").reshape(n, R, Hq * D)
    # the same bits as the one-tile kernel gives: both halves of the rows by themselves (512 rows a
    # call stay below the switch), the second half against a prefix that ends with it
    q = np.array(case["q"], np.uint16).reshape(n, Hq, R, D)
    for first in (0, 512):
        part = dict(case, R=512, a=first, L=first + 512, q=q[:, :, first:first + 512].reshape(-1).tolist())
        one = run(part, 0, expect_kernel="sdpa_mfma").reshape(n, 512, Hq * D)
        assert np.array_equal(got[:, first:first + 512], one)
    # one plane against the oracle: held to the float64 budget of the BF16 probability on every element,
    # like the seeded shapes (with 1024 terms a sum, outputs that cancel to near zero leave the fixture
    # rule in both kernels alike)
    k = np.array(case["k"], np.uint16).reshape(n, Hkv, R, D)
    v = np.array(case["v"], np.uint16).reshape(n, Hkv, R, D)
    plane = dict(case, leading=[], q=q[1].reshape(-1).tolist(), k=k[1].reshape(-1).tolist(), v=v[1].reshape(-1).tolist())
    want = oracle(plane)
    ref64, budget = float64_attention(plane)
    g = datagen.bf16_to_f32(got[1].reshape(-1)).astype(np.float64).reshape(ref64.shape)
    w = datagen.bf16_to_f32(want.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)
    assert np.all(np.abs(w - ref64) <= budget)
    assert len(close_to_oracle(got[1], want)) <= got[1].size // 100000


def test_two_row_tiles_a_wave_with_special_scores_and_values():
    """A workgroup of the two-tile kernel whose rows meet a NaN or infinite score, or whose KV head
    has an infinity in V, forms its rows in the reference's order: same value classes as the oracle
    everywhere, and the bits of the plain case in the KV heads that have nothing special."""
    R, D = 70, 64
    case = random_case(73, (2,), 8, 2, R, D, 100, 20, 20 + R)
    q = np.array(case["q"], np.uint16).reshape(2, 8, R, D).copy()
    k = np.array(case["k"], np.uint16).reshape(2, 2, 100, D).copy()
    v = np.array(case["v"], np.uint16).reshape(2, 2, 100, D).copy()
    k[0, 0, 5, 3] = 0x7F80            # +inf in one feature of one token: scores of +inf / -inf
    q[0, 6, 3, 7] = 0x7FC0            # a NaN row (plane 0, head 6 -> KV head 1)
    v[1, 1, 40, 2] = 0x7F80           # an infinity in V of plane 1, KV head 1
    special = dict(case, q=q.reshape(-1).tolist(), k=k.reshape(-1).tolist(), v=v.reshape(-1).tolist())
    got = run(special, 2, expect_kernel="sdpa_mfma_pair")
    assert close_to_oracle(got, oracle(special)) == []
    g = got.reshape(2, R, 8, D)
    assert np.all((g[0, 3, 6] & 0x7FFF) > 0x7F80)
    plain = run(case, 2).reshape(2, R, 8, D)
    assert np.array_equal(g[1][:, :4], plain[1][:, :4])              # plane 1, KV head 0: untouched by any of it


@pytest.mark.parametrize("R", [6, 20], ids=["decode_kernel", "tiled_kernel_and_guard"])
def test_tail_future_tokens_and_special_v(R):
    """The cache tail and tokens no row may see hold infinities and NaN: results are the
    same bits as with finite values there.  An infinity in a V row that some rows see and
    others do not reaches exactly the rows that see it."""
    case = random_case(5, (2,), 4, 2, R, 16, 24, 4, 8)
    base = run(case, 0)
    k = np.array(case["k"], np.uint16).reshape(2, 2, 24, 16).copy()
    v = np.array(case["v"], np.uint16).reshape(2, 2, 24, 16).copy()
    k[:, :, 8:, :] = 0x7FC0
    v[:, :, 8:, :] = 0x7F80
    tail = dict(case, k=k.reshape(-1).tolist(), v=v.reshape(-1).tolist())
    assert np.array_equal(run(tail, 0, fill=0xFF), base)
    assert np.array_equal(run(tail, 1, fill=0xFF), run(case, 1))
    # token 6 is visible to rows r >= 2 (a + r + 1 > 6) only
    v2 = np.array(case["v"], np.uint16).reshape(2, 2, 24, 16).copy()
    v2[0, 1, 6, 3] = 0x7F80
    part = dict(case, v=v2.reshape(-1).tolist())
    got = run(part, 0)
    want = oracle(part)
    assert close_to_oracle(got, want) == []
    g = got.reshape(2, R, 4, 16)
    assert np.all(g[0, 2:, 2:, 3] == 0x7F80) and np.all((g[0, :2, :, :] & 0x7F80) != 0x7F80)
    assert np.array_equal(g[1], base.reshape(2, R, 4, 16)[1])


@pytest.mark.parametrize("Hkv", [2, 8], ids=["four_heads_share", "four_row_tiles_share"])
@pytest.mark.parametrize("D", [64, 128])
def test_special_scores_where_four_waves_share_the_groups(D, Hkv):
    """Eight query heads on two KV heads (the tiled kernel's four waves = four heads read K and
    V from one LDS ring and fall back to the special-row passes together) or on eight (four
    waves = four row tiles of one head, the last workgroup with waves past the last tile): K
    rows that make scores of +infinity and -infinity, a NaN in one Q row, a row of zero scores."""
    R = 40 if Hkv == 2 else 72
    case = random_case(61, (2,), 8, Hkv, R, D, 100, 20, 20 + R)
    q = np.array(case["q"], np.uint16).reshape(2, 8, R, D).copy()
    k = np.array(case["k"], np.uint16).reshape(2, Hkv, 100, D).copy()
    k[0, 0, 5, 3] = 0x7F80            # +inf in one feature: the score is +inf or -inf by the sign of q
    k[1, 1, 9, 2] = 0xFF80
    q[0, 6, 3, 7] = 0x7FC0            # NaN row (plane 0, head 6, row 3)
    q[1, 1, 30, :] = 0x0000           # all scores 0 for this row
    special = dict(case, q=q.reshape(-1).tolist(), k=k.reshape(-1).tolist())
    got = run(special, 0, expect_kernel="sdpa_mfma")
    want = oracle(special)
    assert close_to_oracle(got, want) == []
    g = got.reshape(2, R, 8, D)
    assert np.all((g[0, 3, 6] & 0x7FFF) > 0x7F80)                    # the NaN row is NaN
    # plane 1, KV head 0 (its query heads) has nothing special: bits equal those of the plain case
    plain = run(case, 0).reshape(2, R, 8, D)
    heads = 8 // Hkv
    keep = np.ones((R, heads), bool)
    if heads > 1:
        keep[30, 1] = False
    assert np.array_equal(g[1][:, :heads][keep], plain[1][:, :heads][keep])


@pytest.mark.parametrize("R,kernel", [(1, "sdpa_decode"), (17, "sdpa_mfma")], ids=["decode_kernel", "tiled_kernel_and_guard"])
def test_more_planes_than_one_grid_holds(R, kernel):
    """65540 planes (a grid axis holds 65535): seven different planes repeated; every plane's
    result is the bits of the same plane in a seven-plane call."""
    n, few = 65540, 7
    small = random_case(77, (few,), 2, 1, R, 16, 20, 3, 3 + R)
    want = run(small, 0, expect_kernel=kernel)
    pick = np.arange(n) % few
    big = dict(small, leading=[n])
    for name, shape in (("q", (few, 2, R, 16)), ("k", (few, 1, 20, 16)), ("v", (few, 1, 20, 16))):
        big[name] = np.array(small[name], np.uint16).reshape(shape)[pick].reshape(-1)
    got = run(big, 0, expect_kernel=kernel)
    assert np.array_equal(got, want[pick])


LONG_DECODE = [((), 8, 2, 1, 64, 2200, 2199, 2200), ((3,), 16, 2, 2, 128, 2100, 2050, 2052),
               ((), 4, 4, 3, 32, 2500, 2400, 2403), ((2,), 8, 1, 1, 64, 4100, 4095, 4096)]


@pytest.mark.parametrize("spec", LONG_DECODE, ids=[str(i) for i in range(len(LONG_DECODE))])
def test_decode_step_against_a_long_prefix_in_shares(spec):
    """Few sequences against a prefix of 64 or more token groups: several workgroups per KV head
    share the groups (statistics, then partial sums, then the join).  Against the oracle with the
    fixture rule and the float64 budget; one case per edge: two rows per head on the diagonal,
    three leading planes, one KV head, a prefix that is a multiple of the share size."""
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(81 + R, lead, Hq, Hkv, R, D, C, a, L)
    q, k, v, o = device_operands(case)
    rc, nbytes, align = iomx.sdpa_workspace(q.view(), k.view(), v.view(), o.view(), a, L)
    assert rc == 0 and nbytes > 0 and align == 256
    for t in (q, k, v, o):
        t.free()
    got = run(case, 0, fill=0xFF, expect_kernel="sdpa_decode")
    want = oracle(case)
    ref64, budget = float64_attention(case)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    w = datagen.bf16_to_f32(want.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)                 # every element inside the float64 budget
    assert np.all(np.abs(w - ref64) <= budget)                 # ... as is the oracle
    assert np.all(np.abs(g - w) <= 2 * budget)
    assert close_to_oracle(got, want) == []                    # and the reference's fixture rule holds


RAGGED_DECODE = [((2,), 8, 2, 1, 64, 500, 499, 500), ((), 32, 4, 1, 64, 490, 485, 486),
                 ((2,), 16, 8, 1, 128, 77, 69, 70), ((), 4, 2, 1, 40, 100, 50, 51),
                 ((), 8, 2, 2, 64, 300, 298, 300), ((2,), 8, 2, 1, 64, 2300, 2210, 2211)]


@pytest.mark.parametrize("spec", RAGGED_DECODE, ids=[str(i) for i in range(len(RAGGED_DECODE))])
def test_decode_step_whose_prefix_ends_inside_a_token_group(spec):
    """A decode step at a position that is not a multiple of 32 (31 of 32 steps of a session): every
    row in use sees the same prefix, and the ragged last group takes the matrix cores with the V of
    its tokens past the prefix taken as zero.  The cache tail holds NaN and infinities (the bits of
    the result do not depend on it), a cache that ends in the group's first token tile is not read
    past its end, and the results hold the fixture rule and the float64 budget against the oracle.
    Cases: the cache ends with the prefix; the group's second tile is not there; D = 128 and a D
    that is no multiple of 16; two rows that both reach the end of the prefix; in shares."""
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(131 + L, lead, Hq, Hkv, R, D, C, a, L)
    n = int(np.prod(lead)) if lead else 1
    k = np.array(case["k"], np.uint16).reshape(n, Hkv, C, D).copy()
    v = np.array(case["v"], np.uint16).reshape(n, Hkv, C, D).copy()
    k[:, :, L:, :] = 0x7FC0
    v[:, :, L:, 0::2] = 0xFF80
    v[:, :, L:, 1::2] = 0x7FC0
    tail = dict(case, k=k.reshape(-1).tolist(), v=v.reshape(-1).tolist())
    got = run(tail, 0, fill=0xFF, expect_kernel="sdpa_decode")
    assert np.array_equal(got, run(case, 0, expect_kernel="sdpa_decode"))
    want = oracle(case)
    ref64, budget = float64_attention(case)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)
    assert close_to_oracle(got, want) == []


KEPT_SCORES = [((2,), 8, 2, 1, 64, 1100, 1049, 1050), ((), 16, 2, 1, 128, 700, 650, 651),
               ((), 8, 2, 2, 64, 900, 800, 802), ((), 16, 1, 1, 64, 1900, 1899, 1900),
               ((), 8, 1, 2, 128, 1800, 1700, 1702), ((), 4, 4, 4, 96, 640, 600, 604)]


@pytest.mark.parametrize("spec", KEPT_SCORES, ids=[str(i) for i in range(len(KEPT_SCORES))])
def test_decode_step_that_keeps_its_scores_between_the_passes(spec):
    """One launch against a prefix of 17 to 63 token groups: more than the K ring holds, so the
    scores of pass 1 stay in LDS and pass 2 reads neither K nor multiplies again.  Cases 0-2 fit
    behind the kernel's own arrays (D = 64 and 128; two rows per head, whose diagonal group takes
    the vector path); cases 3-4 have 16 tile rows in use and 55 or more groups, which fit only as
    per-wave areas that the partial outputs take over (case 4 with the vector path's probabilities
    in the same area); case 5 is D = 96 with four rows.  Against the oracle (fixture rule, float64
    budget), with NaN and infinities in the cache tail, which the result's bits do not depend on."""
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(171 + L, lead, Hq, Hkv, R, D, C, a, L)
    q, k, v, o = device_operands(case)
    rc, nbytes, align = iomx.sdpa_workspace(q.view(), k.view(), v.view(), o.view(), a, L)
    assert rc == 0 and nbytes == 0                                  # one launch, no workspace
    for t in (q, k, v, o):
        t.free()
    n = int(np.prod(lead)) if lead else 1
    kk = np.array(case["k"], np.uint16).reshape(n, Hkv, C, D).copy()
    vv = np.array(case["v"], np.uint16).reshape(n, Hkv, C, D).copy()
    kk[:, :, L:, :] = 0x7FC0
    vv[:, :, L:, :] = 0x7F80
    tail = dict(case, k=kk.reshape(-1).tolist(), v=vv.reshape(-1).tolist())
    got = run(tail, 0, fill=0xFF, expect_kernel="sdpa_decode")
    assert np.array_equal(got, run(case, 0, expect_kernel="sdpa_decode"))
    want = oracle(case)
    ref64, budget = float64_attention(case)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)
    assert close_to_oracle(got, want) == []


@pytest.mark.parametrize("L", [151, 700], ids=["k_ring", "kept_scores"])
def test_decode_step_with_special_scores_among_whole_groups(L):
    """One launch, several token groups that every row sees whole: their statistics and probabilities
    take the short forms, which hold for finite and -infinity scores only; a +infinity score, a NaN
    query row, a KV head whose every score is -infinity, +infinity or NaN, and a head whose scores
    all lie below -1e30 (the stand-in for "no maximum yet" in the short form's exponent arguments)
    must send the wave back to the careful form.  Against the oracle under the fixture rule."""
    Hq, Hkv, R, D, C, a = 8, 2, 1, 64, L + 40, L - 1
    case = random_case(191 + L, (2,), Hq, Hkv, R, D, C, a, L)
    q = np.array(case["q"], np.uint16).reshape(2, Hq, R, D).copy()
    k = np.array(case["k"], np.uint16).reshape(2, Hkv, C, D).copy()
    k[0, 0, 3, 5] = 0x7F80            # +inf or -inf scores of plane 0, heads 0-3, by the sign of q
    q[1, 2, 0, 9] = 0x7FC0            # a NaN row
    k[1, 1, :, :] = 0x0000
    k[1, 1, :L, 0] = 0xFF80           # every score of plane 1, heads 4-7: -inf, +inf or NaN
    q[0, 4:, 0, :] = 0x0000
    q[0, 4:, 0, 0] = 0x5B00           # 2^55 ...
    k[0, 1, :, :] = 0x0000
    k[0, 1, :L, 0] = 0xDB00 + (np.arange(L) % 5).astype(np.uint16)   # ... times about -2^55: scores near -1.6e32
    special = dict(case, q=q.reshape(-1).tolist(), k=k.reshape(-1).tolist())
    qd, kd, vd, od = device_operands(special)
    rc, nbytes, _ = iomx.sdpa_workspace(qd.view(), kd.view(), vd.view(), od.view(), a, L)
    assert rc == 0 and nbytes == 0
    for t in (qd, kd, vd, od):
        t.free()
    got = run(special, 0, expect_kernel="sdpa_decode")
    want = oracle(special)
    assert close_to_oracle(got, want) == []
    g = got.reshape(2, R, Hq, D)
    assert np.all((g[1, 0, 2] & 0x7FFF) > 0x7F80)                        # the NaN row
    w = want.reshape(2, R, Hq, D)
    assert np.array_equal((g[0, 0, 4:] & 0x7F80) == 0x7F80, (w[0, 0, 4:] & 0x7F80) == 0x7F80)
    # the untouched half (plane 1, heads 0-3 except the NaN row) equals the run without special values
    plain = run(case, 0).reshape(2, R, Hq, D)
    assert np.array_equal(g[1, 0, [0, 1, 3]], plain[1, 0, [0, 1, 3]])


@pytest.mark.parametrize("spec,kernel", [(((), 8, 2, 1, 64, 300, 299, 300), "sdpa_decode"),
                                         (((), 8, 2, 1, 128, 700, 699, 700), "sdpa_decode"),
                                         (((), 8, 2, 64, 64, 64, 0, 64), "sdpa_mfma")],
                         ids=["decode", "decode_kept_scores", "prefill"])
def test_a_subnormal_k_against_a_huge_q_is_flushed(spec, kernel):
    """The dot product flushes subnormal operands (src/cpu/sdpa.cpp:57-60).  Sixteen K elements of
    nearly 2^-126 meet q elements of 2^127: unflushed, the products would raise one token's score of
    every row by 4 (D = 64), far outside any tolerance.  The other K elements of those features are
    zeros, so the matrix-core kernels' test for zero exponent fields finds something in every wave
    that meets these features; the rest of K and all of V hold none."""
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(211 + L, lead, Hq, Hkv, R, D, C, a, L)
    q = np.array(case["q"], np.uint16).reshape(1, Hq, R, D).copy()
    k = np.array(case["k"], np.uint16).reshape(1, Hkv, C, D).copy()
    q[:, :, :, 5:21] = 0x7F00         # 2^127 in sixteen features
    k[:, :, :, 5:21] = 0x0000
    k[0, 0, 17, 5:21] = 0x007F        # the largest subnormal, nearly 2^-126: unflushed, +32 on the dot product,
    k[0, 1, L - 3, 5:21] = 0x807F     # +4 (D = 64) on the score and a factor of 55 on that token's weight
    case = dict(case, q=q.reshape(-1).tolist(), k=k.reshape(-1).tolist())
    got = run(case, 0, expect_kernel=kernel)
    want = oracle(case)
    assert close_to_oracle(got, want) == []
    # the check is a sharp one: the same operands with the subnormals made the smallest normal number
    # give visibly different rows
    k2 = k.copy()
    k2[0, 0, 17, 5:21] = 0x0080
    moved = oracle(dict(case, k=k2.reshape(-1).tolist()))
    assert close_to_oracle(moved, want) != []
    ref64, budget = float64_attention(case)                       # (flushes the operands as well)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)


def test_decode_in_shares_with_special_scores_and_values():
    """Special scores that fall into different shares (a +infinity score in the first and the last
    share, a NaN query row, a row of -infinity scores), an infinite V at a token only the second
    row of each head may see, and NaN / infinity in the cache tail."""
    Hq, Hkv, R, D, C, a, L = 8, 2, 2, 64, 2300, 2200, 2202
    case = random_case(91, (2,), Hq, Hkv, R, D, C, a, L)
    q = np.array(case["q"], np.uint16).reshape(2, Hq, R, D).copy()
    k = np.array(case["k"], np.uint16).reshape(2, Hkv, C, D).copy()
    v = np.array(case["v"], np.uint16).reshape(2, Hkv, C, D).copy()
    k[0, 0, 3, 5] = 0x7F80            # +inf or -inf scores by the sign of q, first share
    k[0, 0, 2190, 5] = 0x7F80         # ... and last share
    q[1, 2, 1, 9] = 0x7FC0            # a NaN row
    k[1, 1, :, :] = 0x0000
    k[1, 1, :L, 0] = 0xFF80           # every visible score of KV head 1 of plane 1 is -inf or +inf or NaN
    v[0, 1, 2201, 7] = 0x7F80         # visible to row 1 (a + 1 + 1 = 2202 tokens) but not to row 0
    k[:, :, L:, :] = 0x7FC0
    v[:, :, L:, :] = 0xFF80
    special = dict(case, q=q.reshape(-1).tolist(), k=k.reshape(-1).tolist(), v=v.reshape(-1).tolist())
    got = run(special, 0, expect_kernel="sdpa_decode")
    want = oracle(special)
    assert close_to_oracle(got, want) == []
    g = got.reshape(2, R, Hq, D)
    assert np.all(g[0, 1, 4:, 7] == 0x7F80) and np.all((g[0, 0, 4:, :] & 0x7F80) != 0x7F80)
    assert np.all((g[1, 1, 2] & 0x7FFF) > 0x7F80)


def test_incremental_rows_equal_the_prefill():
    case = random_case(9, (), 4, 2, 7, 8, 7, 0, 7)
    full = run(case, 0)
    for r in range(7):
        c = dict(case, R=1, q=np.array(case["q"], np.uint16).reshape(4, 7, 8)[:, r:r + 1].reshape(-1).tolist())
        c["a"], c["L"] = r, r + 1
        one = run(c, 0)
        assert close_to_oracle(one[0], full[r]) == []


def test_views_and_rejections():
    # q, k, v as windows of larger owners; out a plane of a larger owner
    Hq, Hkv, R, D, C, a, L = 4, 2, 20, 16, 40, 3, 18
    case = random_case(77, (2,), Hq, Hkv, R, D, C, a, L)
    want = oracle(case)
    qo = iomx.DeviceTensor(DT_BF16, (3, Hq, R, D), fill=0x11)
    ko = iomx.DeviceTensor(DT_BF16, (2, Hkv + 1, C, D), fill=0x11)
    vo = iomx.DeviceTensor(DT_BF16, (2, Hkv, C, D), fill=0x11)
    oo = iomx.DeviceTensor(DT_BF16, (4, R, Hq * D), fill=0x11)
    qv = qo.view().slice(0, 1, 2, 1)
    kv = ko.view().slice(1, 1, Hkv, 1)
    ov = oo.view().slice(0, 0, 2, 2)
    qv.from_host(np.array(case["q"], np.uint16).reshape(2, Hq, R, D))
    kv.from_host(np.array(case["k"], np.uint16).reshape(2, Hkv, C, D))
    vo.view().from_host(np.array(case["v"], np.uint16).reshape(2, Hkv, C, D))
    rc, nbytes, _ = iomx.sdpa_workspace(qv, kv, vo.view(), ov, a, L)
    assert rc == 0 and nbytes > 0
    ws = iomx.Buffer(nbytes)
    assert iomx.sdpa(qv, kv, vo.view(), ov, a, L, ws) == 0
    iomx.synchronize()
    assert close_to_oracle(ov.to_host(), want) == []
    assert np.all(oo.view().to_host()[[1, 3]] == 0x1111)
    # admission
    q, k, v, o = qo.view().slice(0, 0, 2, 1), ko.view().slice(1, 0, Hkv, 1), vo.view(), oo.view().slice(0, 0, 2, 1)
    for bad_a, bad_L in ((3, 0), (3, 41), (40, 18), (21, 18)):
        assert iomx.sdpa(q, k, v, o, bad_a, bad_L, ws) == -1
    assert iomx.sdpa(q, k, v, o, a, L, None) == -1                  # the matrix-core path needs its workspace
    assert iomx.sdpa(q, k, v, o, a, L, None, 1) == 0                # the reference-order path does not
    small = iomx.Buffer(512)
    assert iomx.sdpa(q, k, v, o, a, L, small) == -1
    assert iomx.sdpa(q, ko.view(), v, o, a, L, ws) == -1            # Hq % Hkv != 0
    f = [iomx.DeviceTensor(DT_F32, d) for d in ((4, 3, 8), (2, 10, 8), (3, 32))]
    assert iomx.sdpa(f[0].view(), f[1].view(), f[1].view(), f[2].view(), 2, 5, ws) == -2
    iomx.synchronize()
    for t in (qo, ko, vo, oo, *f):
        t.free()
    ws.free()
    small.free()


# -- through the C++ backend, next to the reference CPU backend ---------------------------

@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


def backend_run(dev, case):
    qd, kd, od = shapes(case)
    t = [dev.tensor(DT_BF16, d) for d in (qd, kd, kd, od)]
    t[0].view().from_host(np.array(case["q"], np.uint16).reshape(qd))
    t[1].view().from_host(np.array(case["k"], np.uint16).reshape(kd))
    t[2].view().from_host(np.array(case["v"], np.uint16).reshape(kd))
    token = dev.sdpa(t[0].view(), t[1].view(), t[2].view(), t[3].view(), case["a"], case["L"])
    got = t[3].view().to_host() if token > 0 else None
    for x in t:
        x.close()
    return token, got


@pytest.mark.parametrize("index", range(len(CASES)), ids=[c["label"].replace(" ", "_") for c in CASES])
def test_backend_on_the_reference_fixtures(devices, index):
    cpu, gpu = devices
    case = CASES[index]
    token, got = backend_run(gpu, case)
    assert token > 0, gpu.error()
    assert all_match(got, case) == []
    token, want = backend_run(cpu, case)
    assert token > 0, cpu.error()
    assert close_to_oracle(got, want) == []


def within_budget_of_each_other(case, got, want):
    """Both results inside the float64 budget of the BF16 probability on every element, hence
    within twice that budget of each other."""
    ref64, budget = float64_attention(case)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    w = datagen.bf16_to_f32(want.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget)
    assert np.all(np.abs(w - ref64) <= budget)
    assert np.all(np.abs(g - w) <= 2 * budget)


def test_backend_prefill_then_decode_and_rejections(devices):
    cpu, gpu = devices
    case = random_case(91, (2,), 8, 2, 24, 64, 48, 0, 24)
    outs = [backend_run(dev, case) for dev in (cpu, gpu)]
    assert outs[0][0] > 0 and outs[1][0] > 0
    within_budget_of_each_other(case, outs[1][1], outs[0][1])
    step = dict(case, R=1, a=24, L=25,
                q=np.array(case["q"], np.uint16).reshape(2, 8, 24, 64)[:, :, :1].reshape(-1).tolist())
    outs = [backend_run(dev, step) for dev in (cpu, gpu)]
    assert close_to_oracle(outs[1][1], outs[0][1]) == []
    # a decode step against a long prefix: the backend asks for and passes the workspace of the shares
    far = random_case(93, (), 8, 2, 1, 64, 2200, 2199, 2200)
    outs = [backend_run(dev, far) for dev in (cpu, gpu)]
    assert outs[0][0] > 0 and outs[1][0] > 0
    within_budget_of_each_other(far, outs[1][1], outs[0][1])
    # admission and capability answers are the reference's own
    for bad in (dict(case, L=0), dict(case, L=49), dict(case, a=48), dict(case, a=30)):
        assert backend_run(cpu, bad)[0] == backend_run(gpu, bad)[0] < 0
    for dev in (cpu, gpu):
        f = [dev.tensor(DT_F32, d) for d in ((4, 3, 8), (2, 10, 8), (3, 32))]
        assert dev.sdpa(f[0].view(), f[1].view(), f[1].view(), f[2].view(), 2, 5) < 0
        for x in f:
            x.close()
