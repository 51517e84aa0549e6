"""Above the decode rows: the trellis GEMM chains against the CPU oracle, with the cases and bars of turboexl3
src/hip_tests.zig:704-760 (routed prefill: sampled rows within 5e-3 (f32) / 1.5e-2 (bf16) of rms; rows 0-16 byte-equal
whatever the row count) and src/hip_tests.zig:287-350's dense bars (f32 5e-3, bf16 2.5e-2) past 32 rows."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, make_x, to_f32
from tests.test_gpu_dense import DenseCase
from tests.test_gpu_moe import RefBank, dev_bank, routing

pytestmark = pytest.mark.gpu

F32_BAR = 5e-3
BF16_DENSE_BAR = 2.5e-2
BF16_MOE_BAR = 1.5e-2


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


DENSE = [
    # (in, out, n, codebook, wbits, dtype); out = 384: a workgroup whose last wave has no column
    (512, 256, 64, MCG, 16, torch.float32),
    (512, 384, 64, MUL1, 16, torch.float32),
    (512, 256, 36, MCG, 16, torch.float32),
    (512, 256, 128, MCG, 12, torch.float32),
    (1024, 512, 96, MUL1, 16, torch.float16),
    (2560, 640, 80, MUL1, 16, torch.bfloat16),
    (512, 256, 112, MCG, 16, torch.float32),     # K7: the four-word wide reader
]


@pytest.mark.parametrize("in_f,out_f,n,codebook,wbits,dtype", DENSE)
def test_dense_above_32_rows(oracle, t3, in_f, out_f, n, codebook, wbits, dtype):
    case = DenseCase(oracle, t3, 0xBEEF + in_f + n, in_f, out_f, n, codebook, wbits)
    max_rows = 200
    x_dev, x_f32 = make_x(case.rng, max_rows, in_f, dtype, outliers=True)
    yref = case.ref(x_f32)
    bar = F32_BAR if dtype == torch.float32 else BF16_DENSE_BAR
    worst, first = 0.0, None
    for rows in (33, 64, 65, 200):
        y = t3.linear(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec)
        assert y.shape == (rows, out_f) and y.dtype == dtype
        got = to_f32(y)
        for r in range(rows):
            e = oracle.compare(got[r], yref[r])
            worst = max(worst, e)
            assert e <= bar, f"rows {rows} row {r}: {e:.3e} over the bar {bar}"
        # a row's bytes do not depend on the rows beside it
        if first is None:
            first = bytes_of(y[:33])
        else:
            assert bytes_of(y[:33]) == first, f"rows 0-32 of {rows} rows differ from the 33-row call"
    print(f"dense prefill {in_f}x{out_f} n={n} cb={codebook} {dtype}: worst {worst:.3e} (bar {bar})")


def test_dense_exact_mul1_equals_deferred_within_bar_and_prefill_off_refuses(oracle, t3):
    case = DenseCase(oracle, t3, 77, 512, 256, 48, MUL1)
    x_dev, x_f32 = make_x(case.rng, 40, 512, torch.float32)
    yref = case.ref(x_f32)
    t3.configure(mul1_defer=0)
    try:
        y = to_f32(t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec))
    finally:
        t3.configure()
    for r in range(40):
        assert oracle.compare(y[r], yref[r]) <= F32_BAR
    t3.configure(prefill=0)
    try:
        with pytest.raises(t3.T3Error) as err:
            t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec)
        assert err.value.name == "Exl3EngineNotImplemented"
    finally:
        t3.configure()


MOE = [
    # (hidden, inter, experts, topk, n, codebook, wbits, dtype, defer): src/hip_tests.zig:713-718's list
    (512, 256, 12, 4, 64, MCG, 16, torch.float32, 0),
    (512, 256, 12, 4, 64, MUL1, 16, torch.float32, 1),
    (512, 256, 12, 8, 36, MCG, 12, torch.float32, 0),
    (2560, 640, 16, 10, 48, MUL1, 16, torch.bfloat16, 1),
]


@pytest.mark.parametrize("hidden,inter,experts,topk,n,codebook,wbits,dtype,defer", MOE)
def test_routed_prefill_sampled_rows_and_first_17_rows(oracle, t3, hidden, inter, experts, topk, n, codebook, wbits,
                                                       dtype, defer):
    rng = np.random.default_rng(0x9F1 + hidden + n)
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, codebook, (1 << wbits) - 1)
    dec = t3.Decode(codebook, wbits)
    max_rows = 200 if hidden > 512 else 520
    x_dev, x_f32 = make_x(rng, max_rows, hidden, dtype)
    slots, scores = routing(rng, max_rows, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    bar = F32_BAR if dtype == torch.float32 else BF16_MOE_BAR
    worst, y17 = 0.0, None
    t3.configure(mul1_defer=defer)
    try:
        for rows in (17, 40, 200, 520):
            if rows > max_rows:
                continue
            y = t3.moe(x_dev[:rows].reshape(1, rows, hidden), dbank, d_slots[:rows].reshape(1, rows, topk),
                       d_scores[:rows].reshape(1, rows, topk), dec)
            assert y.shape == (1, rows, hidden) and y.dtype == dtype
            got = to_f32(y).reshape(rows, hidden)
            for r in (0, 1, rows // 2, rows - 1):
                e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r]))
                worst = max(worst, e)
                assert e <= bar, f"rows {rows} row {r}: {e:.3e} over the bar {bar}"
            # the first 17 rows' bytes do not depend on the rows after them (their slots land elsewhere in the order)
            if y17 is None:
                y17 = bytes_of(y[0, :17])
            else:
                assert bytes_of(y[0, :17]) == y17, f"rows 0-16 of {rows} rows differ from the 17-row call"
    finally:
        t3.configure()
    print(f"routed prefill {hidden}x{inter} n={n} cb={codebook} {dtype}: worst {worst:.3e} (bar {bar})")


def test_routed_prefill_clamp_skips_mixed_rates_shared(oracle, t3):
    rng = np.random.default_rng(0x51)
    hidden, inter, experts, topk, rows = 512, 256, 40, 3, 70  # few rows an expert: the 32-row items
    bank = oracle.synth_bank(rng, experts, hidden, inter, 32, 48)
    shared = oracle.synth_bank(rng, 1, hidden, inter, 32, 48)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    ref, sref = RefBank(oracle, bank, MCG, 0xFFFF), RefBank(oracle, shared, MCG, 0xFFFF)
    x_dev, x_f32 = make_x(rng, rows, hidden, torch.float32)
    slots, scores = routing(rng, rows, topk, experts)
    slots[3, 1] = -1
    slots[69, 0] = experts
    slots[5, :] = -1  # a row with no live slot: zeros
    d_slots = torch.from_numpy(slots).cuda().reshape(1, rows, topk)
    d_scores = torch.from_numpy(scores).cuda().reshape(1, rows, topk)
    x3 = x_dev.reshape(1, rows, hidden)
    limit = 1
    y = to_f32(t3.moe_clamped(x3, dbank, d_slots, d_scores, t3.Decode.mcg, limit)).reshape(rows, hidden)
    ys = to_f32(t3.moe_shared_expert(x3, dbank, d_slots, d_scores, t3.Decode.mcg, limit, dshared)).reshape(rows, hidden)
    assert not y[5].any()
    for r in (0, 3, 5, 33, 69):
        routed = ref.row(x_f32[r], slots[r], scores[r], float(limit))
        if r != 5:
            assert oracle.compare(y[r], routed) <= F32_BAR
        both = (routed + sref.slot(0, x_f32[r], float(limit))).astype(np.float32)
        assert oracle.compare(ys[r], both) <= F32_BAR
    # moeWithShared's double rounding, bf16
    xb = x3.to(torch.bfloat16)
    sh = torch.from_numpy((rng.standard_normal((1, rows, hidden)) * 0.1).astype(np.float32)).cuda().to(torch.bfloat16)
    yw = t3.moe_with_shared(xb, dbank, d_slots, d_scores, t3.Decode.mcg, False, sh)
    want = (t3.moe(xb, dbank, d_slots, d_scores, t3.Decode.mcg).to(torch.float32) + sh.to(torch.float32)).to(torch.bfloat16)
    assert bytes_of(yw) == bytes_of(want)
    t3.configure(prefill=0)
    try:
        with pytest.raises(t3.T3Error) as err:
            t3.moe(x3, dbank, d_slots, d_scores, t3.Decode.mcg)
        assert err.value.name == "Exl3EngineNotImplemented"
    finally:
        t3.configure()


@pytest.mark.parametrize("in_f,out_f,n,codebook,dtype", [
    (512, 384, 64, MCG, torch.float32),
    (1024, 512, 48, MUL1, torch.float16),
    (2560, 640, 80, MUL1, torch.bfloat16),
])
def test_dense_w_hat_form_from_512_rows(oracle, t3, in_f, out_f, n, codebook, dtype):
    """From t3_config.dense_gemm_rows rows a dense call decodes W_hat once and multiplies with the library's f16 GEMM
    (the reference's dequant + matmul + finish, src/core/dense.zig:909-922,1290-1302; held to the same bars, as its
    Metal form is in src/core/gpu_test.zig:394-438)."""
    case = DenseCase(oracle, t3, 0xA11 + in_f + n, in_f, out_f, n, codebook)
    rows = 530
    x_dev, x_f32 = make_x(case.rng, rows, in_f, dtype, outliers=True)
    yref = case.ref(x_f32)
    bar = F32_BAR if dtype == torch.float32 else BF16_DENSE_BAR
    assert t3.linear_plan(x_dev, case.d_trellis, case.dec)["path"] == 4  # T3_DENSE_W_HAT_GEMM (few tiles: K parts)
    got = to_f32(t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec))
    t3.configure(dense_gemm_rows=0)
    try:
        fused = to_f32(t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec))
    finally:
        t3.configure()
    worst = 0.0
    for r in range(rows):
        for name, y in (("w_hat", got), ("trellis", fused)):
            e = oracle.compare(y[r], yref[r])
            worst = max(worst, e)
            assert e <= bar, f"{name} form row {r}: {e:.3e} over the bar {bar}"
    print(f"dense W_hat form {in_f}x{out_f} n={n} {dtype}: worst {worst:.3e} (bar {bar})")


@pytest.mark.parametrize("in_f,out_f,n,codebook,wbits,dtype", [
    (512, 384, 64, MCG, 16, torch.float32),
    (1024, 512, 48, MUL1, 16, torch.float16),
    (512, 256, 128, MCG, 12, torch.bfloat16),
])
def test_dense_over_a_resident_w_hat(oracle, t3, in_f, out_f, n, codebook, wbits, dtype):
    """The reference's resident trunk (src/core/dense.zig:1323-1345): the W_hat decoded once and kept serves every later
    call's GEMM; "the kept W_hat is the per-call one byte for byte, and so is every output". Held that way against
    `linear`'s own W_hat form at 40 and 530 rows (and so to the oracle's bars, which that form is held to), with the
    reference's refusals: decode rows never read a W_hat."""
    case = DenseCase(oracle, t3, 0x4E5 + in_f + n, in_f, out_f, n, codebook, wbits)
    w_hat = t3.dequant(case.d_trellis, case.dec)
    x_dev, x_f32 = make_x(case.rng, 530, in_f, dtype, outliers=True)
    bar = F32_BAR if dtype == torch.float32 else BF16_DENSE_BAR
    t3.configure(dense_gemm_rows=33)
    try:
        for rows in (40, 530):
            per_call = t3.linear(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec)
            kept = t3.linear_resident(x_dev[:rows], w_hat, case.d_suh, case.d_svh)
            assert bytes_of(kept) == bytes_of(per_call), f"{rows} rows: the kept W_hat's output differs"
        yref = case.ref(x_f32[:40])
        got = to_f32(kept[:40])
        assert max(oracle.compare(got[r], yref[r]) for r in range(40)) <= bar
    finally:
        t3.configure()
    # a 3-d x, as `linear` takes it
    y3 = t3.linear_resident(x_dev[:80].reshape(2, 40, in_f), w_hat, case.d_suh, case.d_svh)
    assert y3.shape == (2, 40, out_f) and bytes_of(y3[1]) == bytes_of(kept[40:80])
    for bad, name in (
        (lambda: t3.linear_resident(x_dev[:32], w_hat, case.d_suh, case.d_svh), "Exl3EngineNotImplemented"),
        (lambda: t3.linear_resident(x_dev[:40], w_hat[:, :out_f - 64].contiguous(), case.d_suh, case.d_svh), "BadExl3Shape"),
        (lambda: t3.linear_resident(x_dev[:40], w_hat.to(torch.bfloat16), case.d_suh, case.d_svh), "BadExl3Dtype"),
        (lambda: t3.linear_resident(x_dev[:40, :in_f - 128].contiguous(), w_hat, case.d_suh, case.d_svh), "BadExl3Shape"),
    ):
        with pytest.raises(t3.T3Error) as err:
            bad()
        assert err.value.name == name


def test_trellis_gemm_every_live_block_count(oracle, t3):
    """The GEMM's K loop is specialised by the item's live 16-row blocks (1..4 in the 64-row shape, 1..8 in the 128-row
    shape): row counts that end an item at every block count, both codebooks."""
    for codebook, seed in ((MCG, 5), (MUL1, 6)):
        case = DenseCase(oracle, t3, seed, 512, 256, 64, codebook)
        x_dev, x_f32 = make_x(case.rng, 257, 512, torch.float32)
        yref = case.ref(x_f32)
        t3.configure(dense_gemm_rows=0)
        try:
            for rows in (33, 47, 48, 49, 63, 64, 65, 80, 81, 96, 97, 112, 113, 128, 129, 145, 161, 177, 193, 209, 225, 241, 257):
                got = to_f32(t3.linear(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec))
                worst = max(oracle.compare(got[r], yref[r]) for r in range(rows))
                assert worst <= F32_BAR, f"codebook {codebook} rows {rows}: {worst:.3e}"
        finally:
            t3.configure()


def test_routed_prefill_an_expert_past_the_item_cut(oracle, t3):
    """A mean share of 64 rows an expert runs the GEMM shape whose items the route cuts at 96 rows; a skewed routing then
    gives one expert every token (two items: 96 rows and the rest) and leaves others without a row. Every row within the
    bar, and the rows' bytes the same as under a routing of the same tokens that takes the 128-row shape (a row's sums
    depend on its matrix and the K order alone)."""
    rng = np.random.default_rng(0x5CE3)
    hidden, inter, experts, topk, tokens = 512, 256, 16, 8, 128
    bank = oracle.synth_bank(rng, experts, hidden, inter, 48)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, MCG, 0xFFFF)
    x_dev, x_f32 = make_x(rng, 2 * tokens, hidden, torch.float32)
    assert t3.moe_plan(x_dev[:tokens].reshape(1, tokens, hidden), dbank,
                       torch.zeros(1, tokens, topk, dtype=torch.int32, device="cuda"))["item_rows"] == 96
    slots = np.stack([np.concatenate([[0], 1 + rng.permutation(9)[:topk - 1]]) for _ in range(2 * tokens)]).astype(np.int32)
    scores = (0.05 + rng.random((2 * tokens, topk)) * 0.2).astype(np.float32)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    call = lambda n: t3.moe(x_dev[:n].reshape(1, n, hidden), dbank, d_slots[:n].reshape(1, n, topk),
                            d_scores[:n].reshape(1, n, topk), t3.Decode.mcg)
    y = call(tokens)
    got = to_f32(y).reshape(tokens, hidden)
    for r in (0, 63, 95, 96, 97, tokens - 1):
        e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r]))
        assert e <= F32_BAR, f"row {r}: {e:.3e}"
    twice = call(2 * tokens)  # 128 rows an expert on average: the 128-row shape
    assert t3.moe_plan(x_dev.reshape(1, 2 * tokens, hidden), dbank, d_slots.reshape(1, 2 * tokens, topk))["item_rows"] == 128
    assert bytes_of(twice[0, :tokens]) == bytes_of(y[0])


def test_routed_prefill_many_experts_and_wide_topk(oracle, t3):
    """More experts than the route's scan handles in one pass (1024), most of them without a row, and the widest
    top-k (32)."""
    rng = np.random.default_rng(0xE11)
    hidden, inter, experts, topk, rows = 128, 128, 1100, 32, 24
    bank = oracle.synth_bank(rng, experts, hidden, inter, 32)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, MUL1, 0xFFFF)
    x_dev, x_f32 = make_x(rng, rows, hidden, torch.float32)
    slots = np.stack([rng.permutation(experts)[:topk] for _ in range(rows)]).astype(np.int32)
    slots[:, 0] = experts - 1 - np.arange(rows)  # the last experts are used too
    scores = (0.01 + rng.random((rows, topk)) * 0.05).astype(np.float32)
    y = to_f32(t3.moe(x_dev.reshape(1, rows, hidden), dbank, torch.from_numpy(slots).cuda().reshape(1, rows, topk),
                      torch.from_numpy(scores).cuda().reshape(1, rows, topk), t3.Decode.mul1)).reshape(rows, hidden)
    for r in (0, 11, rows - 1):
        assert oracle.compare(y[r], ref.row(x_f32[r], slots[r], scores[r])) <= F32_BAR
