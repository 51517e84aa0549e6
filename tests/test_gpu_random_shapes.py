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


@pytest.mark.parametrize("seed", range(8))
def test_random_routed_calls(oracle, t3, seed):
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
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, codebook, (1 << wbits) - 1)
    dec = t3.Decode(codebook, wbits)
    row_counts = sorted({1, int(rng.integers(2, 17)), int(rng.integers(17, 90))})
    x_dev, x_f32 = make_x(rng, row_counts[-1], hidden, dtype)
    slots, scores = routing(rng, row_counts[-1], topk, experts)
    slots[0, 0] = experts + 5 if rng.integers(0, 2) else slots[0, 0]  # sometimes a skipped id
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    for rows in row_counts:
        args = (x_dev[:rows].reshape(1, rows, hidden), dbank, d_slots[:rows].reshape(1, rows, topk),
                d_scores[:rows].reshape(1, rows, topk), dec)
        y = t3.moe_clamped(*args, limit) if limit else t3.moe(*args)
        got = to_f32(y).reshape(rows, hidden)
        for r in sorted({0, rows // 2, rows - 1}):
            want = ref.row(x_f32[r], slots[r], scores[r], float(limit))
            e = oracle.compare(got[r], want, HALF_ULP[dtype])
            assert e <= MOE_BARS[dtype], (f"hidden {hidden} inter {inter} E {experts} top-{topk} n {n_gu}/{n_dn} w{wbits} "
                                          f"cb {codebook} {dtype} limit {limit} rows {rows} row {r}: {e:.3e}")
