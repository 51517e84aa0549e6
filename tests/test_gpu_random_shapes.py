"""Seeded random draws over everything a call can vary (widths, rate, window, codebook, dtype, rows, top-k, experts,
clamp), small enough for the CPU oracle: each draw's dense projection and routed call within the reference's bars
(src/hip_tests.zig:326,344,483,499), W_hat to the bit. The fixed cases elsewhere pin the shapes the reference lists;
this one walks the combinations between them."""
import numpy as np
import pytest
import torch

from tests.gpu_util import bytes_of, dev_f16_bits, dev_u16, host_u16, make_x, to_f32
from tests.test_gpu_moe import RefBank, dev_bank, routing

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
BARS = {torch.float32: 5e-3, torch.float16: 5e-3, torch.bfloat16: 2.5e-2}
MOE_BARS = {torch.float32: 5e-3, torch.float16: 5e-3, torch.bfloat16: 1.5e-2}
# ref.compareRounded (src/core/ref.zig:206-218): an output stored in a narrower dtype may also differ by that store's
# rounding, half a unit in its last place; at one slot a row (top-1) the f32 reference's own rounding to bf16 already
# measures 1.4-1.8e-2 of rms by the plain measure, so the draws here take the store's rounding out as the reference does
HALF_ULP = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def dense_draw(oracle, t3, seed):
    """One seeded dense projection: its operands on the host and the device, W_hat held to the bit on the way."""
    rng = np.random.default_rng(0xD1CE + seed)
    in_f, out_f = 128 * int(rng.integers(1, 9)), 128 * int(rng.integers(1, 7))
    n = 2 * int(rng.integers(8, 65))
    wbits = int(rng.integers(8, 17))
    codebook = int(rng.integers(0, 2))
    dtype = DTYPES[int(rng.integers(0, 3))]
    mask = (1 << wbits) - 1
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d = {"in": in_f, "out": out_f, "n": n, "wbits": wbits, "codebook": codebook, "dtype": dtype, "mask": mask,
         "trellis": trellis, "suh": suh, "svh": svh, "dec": t3.Decode(codebook, wbits),
         "dev": (dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)),
         "what": f"in {in_f} out {out_f} n {n} w{wbits} cb {codebook} {dtype}"}
    d["w_hat"] = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook, mask)
    assert np.array_equal(host_u16(t3.dequant(d["dev"][0], d["dec"])), d["w_hat"]), d["what"]
    d["row_counts"] = sorted({1, int(rng.integers(2, 17)), int(rng.integers(17, 33)), int(rng.integers(33, 200)), 530})
    d["x_dev"], d["x_f32"] = make_x(rng, d["row_counts"][-1], in_f, dtype, outliers=bool(rng.integers(0, 2)))
    d["ref"] = oracle.project_rows(d["x_f32"], trellis, suh, svh, in_f, out_f, n, codebook, mask, threads=8,
                                   w_hat=d["w_hat"])
    return d


def run_dense(t3, d, rows):
    return t3.linear(d["x_dev"][:rows], *d["dev"], d["dec"])


@pytest.mark.parametrize("seed", range(12))
def test_random_dense_calls(oracle, t3, seed):
    d = dense_draw(oracle, t3, seed)
    first = None
    for rows in d["row_counts"]:
        y = run_dense(t3, d, rows)
        got = to_f32(y)
        worst = max(oracle.compare(got[r], d["ref"][r], HALF_ULP[d["dtype"]]) for r in range(rows))
        assert worst <= BARS[d["dtype"]], f"{d['what']} rows {rows}: {worst:.3e}"
        if rows <= 32:  # a decode row's bytes are those of the row alone
            first = bytes_of(y[0]) if first is None else first
            assert bytes_of(y[0]) == first, f"row 0 at {rows} rows differs from the row alone"


def routed_draw(oracle, t3, seed):
    """One seeded routed call: its operands on the host and the device."""
    rng = np.random.default_rng(0xA0E + seed)
    hidden, inter = 128 * int(rng.integers(1, 6)), 128 * int(rng.integers(1, 5))
    experts = int(rng.integers(1, 20))
    topk = int(rng.integers(1, min(experts, 8) + 1))
    n_gu, n_dn = 2 * int(rng.integers(8, 65)), 2 * int(rng.integers(8, 65))
    wbits = int(rng.integers(8, 17))
    codebook = int(rng.integers(0, 2))
    dtype = DTYPES[int(rng.integers(0, 3))]
    limit = int(rng.integers(0, 9))
    bank = oracle.synth_bank(rng, experts, hidden, inter, n_gu, n_dn)
    d = {"hidden": hidden, "inter": inter, "experts": experts, "topk": topk, "n_gu": n_gu, "n_dn": n_dn, "wbits": wbits,
         "codebook": codebook, "dtype": dtype, "limit": limit, "bank": bank, "dbank": dev_bank(t3, bank),
         "dec": t3.Decode(codebook, wbits)}
    d["row_counts"] = sorted({1, int(rng.integers(2, 17)), int(rng.integers(17, 90))})
    d["x_dev"], d["x_f32"] = make_x(rng, d["row_counts"][-1], hidden, dtype)
    slots, scores = routing(rng, d["row_counts"][-1], topk, experts)
    slots[0, 0] = experts + 5 if rng.integers(0, 2) else slots[0, 0]  # sometimes a skipped id
    d["slots"], d["scores"] = slots, scores
    d["d_slots"], d["d_scores"] = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    d["what"] = (f"hidden {hidden} inter {inter} E {experts} top-{topk} n {n_gu}/{n_dn} w{wbits} cb {codebook} {dtype} "
                 f"limit {limit}")
    return d


def run_routed(t3, d, rows):
    args = (d["x_dev"][:rows].reshape(1, rows, d["hidden"]), d["dbank"], d["d_slots"][:rows].reshape(1, rows, d["topk"]),
            d["d_scores"][:rows].reshape(1, rows, d["topk"]), d["dec"])
    y = t3.moe_clamped(*args, d["limit"]) if d["limit"] else t3.moe(*args)
    return to_f32(y).reshape(rows, d["hidden"])


@pytest.mark.parametrize("seed", range(8))
def test_random_routed_calls(oracle, t3, seed):
    d = routed_draw(oracle, t3, seed)
    ref = RefBank(oracle, d["bank"], d["codebook"], (1 << d["wbits"]) - 1)
    for rows in d["row_counts"]:
        got = run_routed(t3, d, rows)
        for r in sorted({0, rows // 2, rows - 1}):
            want = ref.row(d["x_f32"][r], d["slots"][r], d["scores"][r], float(d["limit"]))
            e = oracle.compare(got[r], want, HALF_ULP[d["dtype"]])
            assert e <= MOE_BARS[d["dtype"]], f"{d['what']} rows {rows} row {r}: {e:.3e}"


def unrounded_table(codebook):
    """Every codeword's weight before the format rounds it to f16, exact in float64: the values the served forms feed the
    matrix cores. MUL1's deferred map: A (1024 + t) + B (src/kernels/hip/common.hpp:95-104; the served form of
    src/core/decode.zig:346). MCG's pair form: the hash's two f16 halves added without the rounding."""
    cw = np.arange(65536, dtype=np.uint64)
    if codebook == 0:
        a, b = float(np.uint16(0x1EEE).view(np.float16)), float(np.uint16(0xC931).view(np.float16))
        h = (cw * 0x83DCD12D) & 0xFFFFFFFF
        t = (h & 0xFF) + ((h >> 8) & 0xFF) + ((h >> 16) & 0xFF) + (h >> 24)
        return a * (1024.0 + t.astype(np.float64)) + b
    p = 0x3B603B60 ^ ((cw * 0xCBAC1FED) & 0x8FFF8FFF)
    half = lambda v: v.astype(np.uint16).view(np.float16).astype(np.float64)
    return half(p & 0xFFFF) + half(p >> 16)


def codeword_matrix(oracle, trellis, in_f, out_f, n):
    """The codeword behind every weight, [in, out]: unpackTile's code positions put where tensorCorePerm puts them."""
    perm = oracle.tensor_core_perm().astype(np.int64)
    t = np.asarray(trellis, dtype=np.uint16).reshape(in_f // 16, out_f // 16, n)
    cw = np.zeros((in_f, out_f), dtype=np.uint16)
    tile = np.zeros(256, dtype=np.uint16)
    for i in range(in_f // 16):
        for j in range(out_f // 16):
            tile[perm] = oracle.unpack_tile(t[i, j], n)
            cw[16 * i:16 * i + 16, 16 * j:16 * j + 16] = tile.reshape(16, 16)
    return cw


def unrounded_weights(oracle, trellis, in_f, out_f, n, codebook, mask, w_hat):
    """float64 [in, out] of `unrounded_table`, checked on the way: rounded to f16 they are the format's W_hat to the bit."""
    w = unrounded_table(codebook)[codeword_matrix(oracle, trellis, in_f, out_f, n) & mask]
    assert np.array_equal(w.astype(np.float16).view(np.uint16), np.asarray(w_hat).reshape(in_f, out_f))
    return w


class UnroundedBank(RefBank):
    """The routed chain with every weight as the served form makes it (`unrounded_table`), never rounded to f16. Everything
    else as RefBank: the oracle's prepare and finish around an inner product taken in float64, z rounded to f16 once."""

    def __init__(self, oracle, bank, codebook, mask):
        super().__init__(oracle, bank, codebook, mask)
        self.unrounded = {}

    def project(self, which, e, x):
        b = self.b
        t, suh, svh, in_f, out_f, n = {
            "gate": (b.gate_t, b.gate_suh, b.gate_svh, b.hidden, b.inter, b.n_gu),
            "up": (b.up_t, b.up_suh, b.up_svh, b.hidden, b.inter, b.n_gu),
            "down": (b.down_t, b.down_suh, b.down_svh, b.inter, b.hidden, b.n_dn)}[which]
        key = (which, e)
        if key not in self.unrounded:
            self.unrounded[key] = unrounded_weights(self.o, t[e], in_f, out_f, n, self.cb, self.mask, self._what(which, e))
        xp = self.o.prepare_input(x, suh[e]).astype(np.float64)
        z = (xp @ self.unrounded[key]).astype(np.float16).astype(np.float32)
        return self.o.finish_output(z, svh[e])


# Draws of a wider walk (500 seeds of each kind) where some row of a call sat at or over the reference's bar against
# format.project's chain while the GEMV fed both codebooks unrounded: ten draws, each a few rows of one or two row counts,
# none above 1.4 x the bar. Two things put a row there, and the tests below hold each draw to the statement that is true
# of it.
#   Unrounded weights. The GEMV feeds MUL1 as the deferred map A h + B (served: the reference's own choice for its
#   kernels, src/core/decode.zig:346, src/kernels/hip/common.hpp:95-104, held there to the same bars at its own shapes,
#   src/hip_tests.zig:450-458,483) and, where t3_config.mcg_pair is set (not by default), MCG as its hashed pair, where
#   format.project rounds every weight to f16. Half an f16 step a weight moves z by ~1.4e-4 of its size, which flips the
#   f16 rounding of a fifth of z's values, and those flips are what the measure sees. On every row: the f16-weight forms
#   (MCG as served; MUL1 with mul1_defer = 0) within the bars of format.project's chain; the unrounded forms within the
#   bars of the same chain with unrounded weights (what the forms define), and within 1.5 x the bars of format.project's.
#   The result's own resolution. y is an f16 value (format.project's last statement rounds it), one f16 step of an
#   element above 5.1 x the row's rms is more than 5e-3 of that rms, and a chain with three f16 rounding points flips a
#   step wherever a sum lands within an f32 rounding of a tie. The dense draws hold every element within the bar or one
#   f16 step of the oracle's value, with the exact weights of the W_hat form as well as with the unrounded ones.
DEFERRED_SLACK = 1.5
ROUTED_AT_THE_BAR = [11, 59, 66, 83, 305, 335, 405]
DENSE_AT_THE_BAR = [117, 122, 445]


@pytest.mark.parametrize("seed", ROUTED_AT_THE_BAR)
def test_routed_draws_where_unrounded_weights_sit_at_the_bar(oracle, t3, seed):
    d = routed_draw(oracle, t3, seed)
    mask = (1 << d["wbits"]) - 1
    exact, unrounded = RefBank(oracle, d["bank"], d["codebook"], mask), UnroundedBank(oracle, d["bank"], d["codebook"], mask)
    bar, half = MOE_BARS[d["dtype"]], HALF_ULP[d["dtype"]]
    most = d["row_counts"][-1]
    mcg = d["codebook"] == 1
    want = [exact.row(d["x_f32"][r], d["slots"][r], d["scores"][r], float(d["limit"])) for r in range(most)]
    want_unr = [unrounded.row(d["x_f32"][r], d["slots"][r], d["scores"][r], float(d["limit"])) for r in range(most)]
    for rows in d["row_counts"]:
        served = run_routed(t3, d, rows)
        # the other form of the draw's codebook: MUL1 decoded weight by weight, MCG's pair fed unrounded
        t3.configure(**({"mcg_pair": 1} if mcg else {"mul1_defer": 0}))
        try:
            other = run_routed(t3, d, rows)
        finally:
            t3.configure()
        exact_form, loose_form = (served, other) if mcg else (other, served)
        # above 16 rows the prefill chain decodes MCG to the format's f16 weights whatever mcg_pair says; MUL1 keeps
        # the deferred map there
        loose_is_unrounded = (not mcg) or rows <= 16
        for r in range(rows):
            e = oracle.compare(exact_form[r], want[r], half)
            assert e <= bar, f"f16 weights, {d['what']} rows {rows} row {r}: {e:.3e}"
            e = oracle.compare(loose_form[r], (want_unr if loose_is_unrounded else want)[r], half)
            assert e <= bar, f"unrounded form against the chain with its own weights, {d['what']} rows {rows} row {r}: {e:.3e}"
            e = oracle.compare(loose_form[r], want[r], half)
            assert e <= DEFERRED_SLACK * bar, f"unrounded form against format.project, {d['what']} rows {rows} row {r}: {e:.3e}"


@pytest.mark.parametrize("seed", DENSE_AT_THE_BAR)
def test_dense_draws_where_one_f16_step_passes_the_bar(oracle, t3, seed):
    d = dense_draw(oracle, t3, seed)
    assert d["dtype"] == torch.float32, "these draws give y as the f16 values themselves"
    bar = BARS[d["dtype"]]
    ref = d["ref"]
    rms = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    step = np.spacing(np.maximum(np.abs(ref), np.float32(2.0 ** -14)).astype(np.float16)).astype(np.float64)
    for rows in d["row_counts"]:
        for form in ({}, {"mcg_pair": 1}, {"mul1_defer": 0}, {"dense_gemm_rows": 0}):
            t3.configure(**form)
            try:
                got = to_f32(run_dense(t3, d, rows))
            finally:
                t3.configure()
            assert np.array_equal(got, got.astype(np.float16).astype(np.float32)), "y is not f16-valued"
            off = np.abs(got.astype(np.float64) - ref[:rows])
            ok = (off <= bar * rms[:rows]) | (off <= step[:rows])
            assert ok.all(), f"{d['what']} rows {rows} {form}: an element beyond the bar and beyond one f16 step"
            worst = max(oracle.compare(got[r], ref[r]) for r in range(rows))
            assert worst <= DEFERRED_SLACK * bar, f"{d['what']} rows {rows} {form}: {worst:.3e}"
