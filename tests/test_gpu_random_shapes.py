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


@pytest.mark.parametrize("seed", range(12))
def test_random_dense_calls(oracle, t3, seed):
    rng = np.random.default_rng(0xD1CE + seed)
    in_f, out_f = 128 * int(rng.integers(1, 9)), 128 * int(rng.integers(1, 7))
    n = 2 * int(rng.integers(8, 65))
    wbits = int(rng.integers(8, 17))
    codebook = int(rng.integers(0, 2))
    dtype = DTYPES[int(rng.integers(0, 3))]
    mask = (1 << wbits) - 1
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    dec = t3.Decode(codebook, wbits)
    w_hat = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook, mask)
    assert np.array_equal(host_u16(t3.dequant(d_t, dec)), w_hat), (in_f, out_f, n, wbits, codebook)
    row_counts = sorted({1, int(rng.integers(2, 17)), int(rng.integers(17, 33)), int(rng.integers(33, 200)), 530})
    x_dev, x_f32 = make_x(rng, row_counts[-1], in_f, dtype, outliers=bool(rng.integers(0, 2)))
    ref = oracle.project_rows(x_f32, trellis, suh, svh, in_f, out_f, n, codebook, mask, threads=8, w_hat=w_hat)
    first = None
    for rows in row_counts:
        y = t3.linear(x_dev[:rows], d_t, d_suh, d_svh, dec)
        got = to_f32(y)
        worst = max(oracle.compare(got[r], ref[r], HALF_ULP[dtype]) for r in range(rows))
        assert worst <= BARS[dtype], f"in {in_f} out {out_f} n {n} w{wbits} cb {codebook} {dtype} rows {rows}: {worst:.3e}"
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


class UnroundedMul1Bank(RefBank):
    """The routed chain with MUL1's weights as the deferred map makes them: w = A (1024 + t) + B, never rounded to f16
    (src/kernels/hip/common.hpp:95-104; the served form of src/core/decode.zig:346). Everything else as RefBank: the
    oracle's prepare and finish around an inner product taken in float64, z rounded to f16 once. t comes back out of the
    oracle's bit-exact W_hat: the codebook's f16 values are distinct for distinct t (their spacing, A, is wider than an
    f16 step anywhere below 4)."""

    A, B = float(np.uint16(0x1EEE).view(np.float16)), float(np.uint16(0xC931).view(np.float16))

    def __init__(self, oracle, bank, mask):
        super().__init__(oracle, bank, 0, mask)
        cw = np.arange(65536, dtype=np.uint64)
        h = (cw * 0x83DCD12D) & 0xFFFFFFFF
        t = (h & 0xFF) + ((h >> 8) & 0xFF) + ((h >> 16) & 0xFF) + (h >> 24)
        bits = oracle.codebook_table(0)
        self.t_of_bits = np.full(65536, -1, dtype=np.int64)
        self.t_of_bits[bits] = t.astype(np.int64)
        assert np.array_equal(self.t_of_bits[bits], t.astype(np.int64)), "MUL1's f16 values collide over t"
        self.unrounded = {}

    def project(self, which, e, x):
        b = self.b
        suh, svh = {"gate": (b.gate_suh, b.gate_svh), "up": (b.up_suh, b.up_svh), "down": (b.down_suh, b.down_svh)}[which]
        key = (which, e)
        if key not in self.unrounded:
            t = self.t_of_bits[self._what(which, e)]
            assert (t >= 0).all()
            self.unrounded[key] = self.A * (1024.0 + t.astype(np.float64)) + self.B
        xp = self.o.prepare_input(x, suh[e]).astype(np.float64)
        z = (xp @ self.unrounded[key]).astype(np.float16).astype(np.float32)
        return self.o.finish_output(z, svh[e])


# Draws of a wider walk (240 seeds) that the served MUL1 form, the deferred map, left at or over the reference's bar on
# some row while the exact-weight form (mul1_defer = 0) stayed well inside: seed 59 (f32) measured 5.1e-3 against 5e-3,
# 2.4e-3 exact; seeds 11 and 66 (bf16) sit at the bar by the plain measure, where the output's own rounding to bf16
# already measures 1.4-1.8e-2. The deferred map feeds A h + B unrounded where format.project rounds every weight to f16,
# as the reference's own kernels do (src/core/decode.zig:346, src/kernels/hip/common.hpp:95-104), and the reference
# holds that form to the same bars at its own shapes (src/hip_tests.zig:450-458,483). Here, on every row:
#   the exact form: within the reference's bars of format.project's chain;
#   the served form: within the same bars of the chain with unrounded weights (what the form defines), and within one and
#   a half times the bars of format.project's chain (measured worst: 5.1e-3 f32): the distance between the two chains is
#   rounding flips of f16 values, not an error of the kernels.
DEFERRED_SLACK = 1.5


@pytest.mark.parametrize("seed", [11, 59, 66])
def test_routed_draws_where_the_deferred_map_sits_at_the_bar(oracle, t3, seed):
    d = routed_draw(oracle, t3, seed)
    assert d["codebook"] == 0, "these draws are MUL1's"
    mask = (1 << d["wbits"]) - 1
    exact, unrounded = RefBank(oracle, d["bank"], 0, mask), UnroundedMul1Bank(oracle, d["bank"], mask)
    bar, half = MOE_BARS[d["dtype"]], HALF_ULP[d["dtype"]]
    rows = d["row_counts"][-1]
    want = [exact.row(d["x_f32"][r], d["slots"][r], d["scores"][r], float(d["limit"])) for r in range(rows)]
    want_unr = [unrounded.row(d["x_f32"][r], d["slots"][r], d["scores"][r], float(d["limit"])) for r in range(rows)]
    served = run_routed(t3, d, rows)
    t3.configure(mul1_defer=0)
    try:
        exact_form = run_routed(t3, d, rows)
    finally:
        t3.configure()
    for r in range(rows):
        e = oracle.compare(exact_form[r], want[r], half)
        assert e <= bar, f"exact form, {d['what']} row {r}: {e:.3e}"
        e = oracle.compare(served[r], want_unr[r], half)
        assert e <= bar, f"served form against the unrounded-weight chain, {d['what']} row {r}: {e:.3e}"
        e = oracle.compare(served[r], want[r], half)
        assert e <= DEFERRED_SLACK * bar, f"served form against format.project, {d['what']} row {r}: {e:.3e}"
