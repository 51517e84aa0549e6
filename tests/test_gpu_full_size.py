"""The benchmark configurations at their full sizes: decoded weights bit-exact, sampled rows (and, where a whole row is
too much for the CPU oracle, sampled 128-column output blocks, which are independent of the rest of the row) within
the reference's bars, and the size-independent byte equalities."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, host_u16, make_x, to_f32
from tests.test_gpu_moe import RefBank, dev_bank

pytestmark = pytest.mark.gpu

F32_BAR, BF16_DENSE_BAR, BF16_MOE_BAR = 5e-3, 2.5e-2, 1.5e-2


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def block_ref(oracle, trellis, suh, svh, x_f32, in_f, n, codebook, blk):
    """Output columns [128 blk, 128 blk + 128) of format.project: the block's own 8 tile columns and svh slice."""
    sub = np.ascontiguousarray(trellis[:, 8 * blk:8 * blk + 8, :])
    return oracle.project_rows(x_f32, sub, suh, np.ascontiguousarray(svh[128 * blk:128 * blk + 128]), in_f, 128, n,
                               codebook, 0xFFFF, threads=8)


def test_config1_cpu_case_2048_k4_one_row(oracle, t3):
    # the reference's own CPU-runnable case: in = out = 2048 at K4, scale vectors sign x N(1, 0.1), one f16 row; the whole
    # output against format.project, both codebooks, and W_hat to the bit
    in_f = out_f = 2048
    n = 64
    rng = np.random.default_rng(0xC1)
    trellis = rng.integers(0, 65536, (in_f // 16, out_f // 16, n), dtype=np.uint16)
    sign = lambda m: rng.choice(np.array([-1.0, 1.0], dtype=np.float32), m)
    suh = (sign(in_f) * rng.normal(1.0, 0.1, in_f)).astype(np.float16).view(np.uint16)
    svh = (sign(out_f) * rng.normal(1.0, 0.1, out_f) / np.sqrt(in_f)).astype(np.float16).view(np.uint16)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, 1, in_f, torch.float16)
    for codebook, dec in ((MCG, t3.Decode.mcg), (MUL1, t3.Decode.mul1)):
        w_hat = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook)
        assert np.array_equal(host_u16(t3.dequant(d_t, dec)), w_hat)
        ref = oracle.project_rows(x_f32, trellis, suh, svh, in_f, out_f, n, codebook, 0xFFFF, threads=8, w_hat=w_hat)
        y = t3.linear(x_dev, d_t, d_suh, d_svh, dec)
        e = oracle.compare(to_f32(y)[0], ref[0], 2.0 ** -11)
        assert e <= F32_BAR, f"codebook {codebook}: {e:.3e}"
        assert bytes_of(y) == bytes_of(t3.linear_chain(x_dev, d_t, d_suh, d_svh, dec)), "one launch differs from the chain"


@pytest.mark.parametrize("k", [3, 4, 5])
def test_config2_qkv_shape_rows_1_4_16_32(oracle, t3, k):
    in_f, out_f, n = 4096, 12288, 16 * k
    rng = np.random.default_rng(0xC2 + k)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    w_hat = oracle.reconstruct_inner(trellis, in_f, out_f, n, MCG)
    assert np.array_equal(host_u16(t3.dequant(d_t, t3.Decode.mcg)), w_hat), "W_hat is not bit-exact at full size"
    x_dev, x_f32 = make_x(rng, 32, in_f, torch.float16, outliers=True)
    ref = oracle.project_rows(x_f32, trellis, suh, svh, in_f, out_f, n, MCG, 0xFFFF, threads=8, w_hat=w_hat)
    alone = t3.linear(x_dev[:1], d_t, d_suh, d_svh, t3.Decode.mcg)
    for rows in (1, 4, 16, 32):
        y = t3.linear(x_dev[:rows], d_t, d_suh, d_svh, t3.Decode.mcg)
        got = to_f32(y)
        for r in range(rows):
            e = oracle.compare(got[r], ref[r], 2.0 ** -11)  # f16 outputs: half an ulp of the store on top of the bar
            assert e <= F32_BAR, f"K{k} rows {rows} row {r}: {e:.3e}"
        assert bytes_of(y[0]) == bytes_of(alone[0]), "row 0 differs from the row alone"


def test_config2_qkv_shape_codebook_forms(oracle, t3):
    # The GEMV's other codebook forms at the q|k|v shape, K4, rows 1 and 32, held to the same bar, the one launch still
    # equal to its chain. Served by default: MCG as the format's f16 weight, MUL1's affine map applied once an output
    # (mul1_defer, the reference's own kernels' form, src/kernels/hip/common.hpp:95-104). Here: every weight the format's
    # f16 value for both codebooks (mul1_defer off), and MCG's hashed pair fed unrounded (mcg_pair on: this library's own
    # opt-in form, which differs from format.project's rounded weight in the last bits of a product).
    in_f, out_f, n = 4096, 12288, 64
    rng = np.random.default_rng(0xC2E)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, 32, in_f, torch.float16, outliers=True)
    refs = {}
    for cfg, books in (({"mcg_pair": 0, "mul1_defer": 0}, ((MCG, t3.Decode.mcg), (MUL1, t3.Decode.mul1))),
                       ({"mcg_pair": 1}, ((MCG, t3.Decode.mcg),))):
        t3.configure(**cfg)
        try:
            for codebook, dec in books:
                if codebook not in refs:
                    w_hat = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook)
                    refs[codebook] = oracle.project_rows(x_f32, trellis, suh, svh, in_f, out_f, n, codebook, 0xFFFF,
                                                         threads=8, w_hat=w_hat)
                ref = refs[codebook]
                for rows in (1, 32):
                    y = t3.linear(x_dev[:rows], d_t, d_suh, d_svh, dec)
                    got = to_f32(y)
                    worst = max(oracle.compare(got[r], ref[r], 2.0 ** -11) for r in range(rows))
                    assert worst <= F32_BAR, f"{cfg} codebook {codebook} rows {rows}: {worst:.3e}"
                    if rows == 1:
                        assert bytes_of(y) == bytes_of(t3.linear_chain(x_dev[:1], d_t, d_suh, d_svh, dec))
        finally:
            t3.configure()


def test_config5_lm_head_k6_rows_1_and_256(oracle, t3):
    in_f, out_f, n = 4096, 151936, 96
    rng = np.random.default_rng(0xC5)
    trellis = rng.integers(0, 65536, (in_f // 16, out_f // 16, n), dtype=np.uint16)
    _, suh, svh = oracle.synth_linear(rng, in_f, 128, n)
    svh = np.tile(svh, out_f // 128)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, 256, in_f, torch.bfloat16)
    y1 = to_f32(t3.linear(x_dev[:1], d_t, d_suh, d_svh, t3.Decode.mul1))
    y256 = to_f32(t3.linear(x_dev, d_t, d_suh, d_svh, t3.Decode.mul1))
    for blk in (0, 1, 593, out_f // 128 - 1):
        ref = block_ref(oracle, trellis, suh, svh, x_f32[[0, 100, 255]], in_f, n, MUL1, blk)
        cols = slice(128 * blk, 128 * blk + 128)
        assert oracle.compare(y1[0, cols], ref[0]) <= BF16_DENSE_BAR
        for i, r in enumerate((0, 100, 255)):
            assert oracle.compare(y256[r, cols], ref[i]) <= BF16_DENSE_BAR, (blk, r)


def test_config5_dense_4096_rows_w_hat_form(oracle, t3):
    in_f, out_f, n, rows = 4096, 14336, 64, 4096
    rng = np.random.default_rng(0xC55)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, rows, in_f, torch.bfloat16)
    y = t3.linear(x_dev, d_t, d_suh, d_svh, t3.Decode.mcg)
    sample = [0, 1, 2047, 4095]
    got = to_f32(y[sample])
    for blk in (0, 55, out_f // 128 - 1):
        ref = block_ref(oracle, trellis, suh, svh, x_f32[sample], in_f, n, MCG, blk)
        for i in range(len(sample)):
            assert oracle.compare(got[i, 128 * blk:128 * blk + 128], ref[i]) <= BF16_DENSE_BAR, (blk, sample[i])


def test_config5_shape_few_rows_on_the_trellis_gemm(oracle, t3):
    # few rows decode the matrix once: the launch shares the tile rows out into K parts (eight at 64 and at 128 rows here,
    # one at 600) and one item's column blocks go round all the dies; sampled blocks against the oracle either way
    in_f, out_f, n = 4096, 14336, 64
    rng = np.random.default_rng(0xC56)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, 600, in_f, torch.bfloat16)
    t3.configure(dense_gemm_rows=0)  # keep 600 rows on the trellis GEMM
    try:
        for rows, sample in ((64, [0, 33, 63]), (128, [0, 70, 127]), (600, [0, 300, 599])):
            got = to_f32(t3.linear(x_dev[:rows], d_t, d_suh, d_svh, t3.Decode.mcg)[sample])
            for blk in (0, 57, out_f // 128 - 1):
                ref = block_ref(oracle, trellis, suh, svh, x_f32[sample], in_f, n, MCG, blk)
                for i in range(len(sample)):
                    e = oracle.compare(got[i, 128 * blk:128 * blk + 128], ref[i])
                    assert e <= BF16_DENSE_BAR, (rows, blk, sample[i], e)
    finally:
        t3.configure()


def test_config5_shape_rows_alone_configuration(oracle, t3):
    # The reference's own GEMM holds rows 0-16 of a 40-, 129- or 200-row call to the bytes of the 17-row call
    # (src/hip_tests.zig:866-880). Here the served launch shape follows the rows (the GEMV up to 32, then eight K parts at
    # 64 rows of this shape, two at 300, the W_hat form at 600), so those bytes may differ between row counts;
    # dense_rows_alone = 1 sends every call above 16 rows to the trellis GEMM with one K part and gives the reference's
    # invariant back, at its own row counts and beyond.
    in_f, out_f, n = 4096, 14336, 64
    rng = np.random.default_rng(0xC57)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, 600, in_f, torch.bfloat16)
    plans = {rows: t3.linear_plan(x_dev[:rows], d_t, t3.Decode.mcg) for rows in (17, 64, 300, 600)}
    assert [plans[r]["k_slices"] for r in (64, 300, 600)] == [8, 2, 1] and plans[600]["path"] == 4
    assert plans[17]["path"] == 2  # the GEMV's chain
    t3.configure(dense_rows_alone=1)
    try:
        first = None
        for rows in (17, 40, 129, 200, 33, 64, 300, 600):
            plan = t3.linear_plan(x_dev[:rows], d_t, t3.Decode.mcg)
            assert (plan["path"], plan["k_slices"]) == (3, 1), rows
            y = t3.linear(x_dev[:rows], d_t, d_suh, d_svh, t3.Decode.mcg)
            first = bytes_of(y[:17]) if first is None else first
            assert bytes_of(y[:17]) == first, f"rows 0-16 of {rows} rows differ from the 17-row call"
        got = to_f32(y[[0, 32, 599]])
        for blk in (0, 57, out_f // 128 - 1):
            ref = block_ref(oracle, trellis, suh, svh, x_f32[[0, 32, 599]], in_f, n, MCG, blk)
            for i in range(3):
                assert oracle.compare(got[i, 128 * blk:128 * blk + 128], ref[i]) <= BF16_DENSE_BAR
        # decode rows keep the GEMV under the switch
        assert t3.linear_plan(x_dev[:16], d_t, t3.Decode.mcg)["path"] == 2
    finally:
        t3.configure()


def test_many_rows_dense_and_routed(oracle, t3):
    # long prefill chunks: 20,000 dense rows on both forms above 32 rows, 6,000 routed tokens; sampled rows (the first, the
    # last, the item boundaries' neighbours) against the oracle
    in_f, out_f, n, rows = 1024, 512, 48, 20000
    rng = np.random.default_rng(0xB16)
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    x_dev, x_f32 = make_x(rng, rows, in_f, torch.bfloat16)
    sample = [0, 127, 128, 9999, rows - 129, rows - 1]
    ref = oracle.project_rows(x_f32[sample], trellis, suh, svh, in_f, out_f, n, MUL1, 0xFFFF, threads=8)
    for gemm_rows in (512, 0):
        t3.configure(dense_gemm_rows=gemm_rows)
        try:
            got = to_f32(t3.linear(x_dev, d_t, d_suh, d_svh, t3.Decode.mul1)[sample])
        finally:
            t3.configure()
        for i, r in enumerate(sample):
            e = oracle.compare(got[i], ref[i])
            assert e <= BF16_DENSE_BAR, f"dense_gemm_rows {gemm_rows} row {r}: {e:.3e}"
    experts, hidden, inter, topk, tokens = 16, 512, 256, 6, 6000
    bank = oracle.synth_bank(rng, experts, hidden, inter, 64)
    dbank = dev_bank(t3, bank)
    rb = RefBank(oracle, bank, MCG, 0xFFFF)
    xm_dev, xm_f32 = make_x(rng, tokens, hidden, torch.float32)
    slots, scores = routing_softmax(rng, tokens, topk, experts)
    y = t3.moe(xm_dev.reshape(1, tokens, hidden), dbank, torch.from_numpy(slots).cuda().reshape(1, tokens, topk),
               torch.from_numpy(scores).cuda().reshape(1, tokens, topk), t3.Decode.mcg)
    got = to_f32(y).reshape(tokens, hidden)
    for r in (0, 1, 2999, tokens - 2, tokens - 1):
        e = oracle.compare(got[r], rb.row(xm_f32[r], slots[r], scores[r]))
        assert e <= F32_BAR, f"token {r}: {e:.3e}"


def routing_softmax(rng, tokens, topk, experts):
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    slots = np.argsort(-logits, axis=1)[:, :topk].astype(np.int32)
    top = np.take_along_axis(logits, slots, axis=1)
    w = np.exp(top - top.max(axis=1, keepdims=True))
    return slots, (w / w.sum(axis=1, keepdims=True)).astype(np.float32)


def test_config3_routed_decode_with_shared_expert(oracle, t3):
    experts, hidden, inter, n, topk, limit = 512, 2048, 512, 48, 10, 7
    rng = np.random.default_rng(0xC3)
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    shared = oracle.synth_bank(rng, 1, hidden, inter, n)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    ref, sref = RefBank(oracle, bank, MCG, 0xFFFF), RefBank(oracle, shared, MCG, 0xFFFF)
    x_dev, x_f32 = make_x(rng, 8, hidden, torch.bfloat16)
    slots, scores = routing_softmax(rng, 8, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    for tokens in (1, 8):
        y = t3.moe_shared_expert(x_dev[:tokens].reshape(1, tokens, hidden), dbank, d_slots[:tokens].reshape(1, tokens, topk),
                                 d_scores[:tokens].reshape(1, tokens, topk), t3.Decode.mcg, limit, dshared)
        got = to_f32(y).reshape(tokens, hidden)
        for r in range(tokens):
            want = (ref.row(x_f32[r], slots[r], scores[r], float(limit)) + sref.slot(0, x_f32[r], float(limit))).astype(np.float32)
            e = oracle.compare(got[r], want)
            assert e <= BF16_MOE_BAR, f"{tokens} tokens row {r}: {e:.3e}"
        if tokens == 1:
            first = bytes_of(y[0, 0])
        else:
            assert bytes_of(y[0, 0]) == first, "row 0 of 8 tokens differs from the row alone"


def test_reference_workload_widths_2560_by_640(oracle, t3):
    # The reference's own published workload (docs/models/qwen38/results.md:278-284): hidden 2560, expert width 640, top-10,
    # bf16, MUL1: 160 and 40 input tile rows, a K partition none of the benchmark configurations has (twenty 128-blocks of
    # the hidden width in five K slices, five of the expert width in two). On 24 of its 512 experts so the CPU side stays
    # small: the decode chain at 1 and 4 rows and the prefill chain at 40 rows against ref.moeRow, a row's bytes those of
    # the row alone, the launch forms equal; and one dense projection of the same widths.
    experts, hidden, inter, n, topk = 24, 2560, 640, 64, 10
    rng = np.random.default_rng(0x2560)
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, MUL1, 0xFFFF)
    x_dev, x_f32 = make_x(rng, 40, hidden, torch.bfloat16)
    slots, scores = routing_softmax(rng, 40, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    plan = t3.moe_plan(x_dev[:1].reshape(1, 1, hidden), dbank, d_slots[:1].reshape(1, 1, topk))
    assert (plan["k_slices_gu"], plan["k_slices_dn"]) == (5, 2), plan
    call = lambda rows: t3.moe(x_dev[:rows].reshape(1, rows, hidden), dbank, d_slots[:rows].reshape(1, rows, topk),
                               d_scores[:rows].reshape(1, rows, topk), t3.Decode.mul1)
    want = [ref.row(x_f32[r], slots[r], scores[r], 0.0) for r in (0, 1, 2, 3, 39)]
    alone = call(1)
    for rows in (1, 4, 40):
        y = call(rows)
        got = to_f32(y).reshape(rows, hidden)
        for i, r in enumerate((0, 1, 2, 3, 39)):
            if r < rows:
                e = oracle.compare(got[r], want[i], 2.0 ** -8)
                assert e <= BF16_MOE_BAR, f"{rows} rows row {r}: {e:.3e}"
        if rows <= 16:
            assert bytes_of(y[0, 0]) == bytes_of(alone[0, 0]), "row 0 differs from the row alone"
            for form in (3, 8):
                t3.configure(decode_form=form)
                try:
                    assert bytes_of(call(rows)) == bytes_of(y), f"form {form} differs at {rows} rows"
                finally:
                    t3.configure()
    # dense, the same widths both ways (the partition of a small matrix: four tiles a load)
    for in_f, out_f in ((2560, 640), (640, 2560)):
        trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
        d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
        xd_dev, xd_f32 = make_x(rng, 4, in_f, torch.bfloat16)
        yref = oracle.project_rows(xd_f32, trellis, suh, svh, in_f, out_f, n, MUL1, 0xFFFF, threads=8)
        for rows in (1, 4):
            y = t3.linear(xd_dev[:rows], d_t, d_suh, d_svh, t3.Decode.mul1)
            assert bytes_of(y) == bytes_of(t3.linear_chain(xd_dev[:rows], d_t, d_suh, d_svh, t3.Decode.mul1))
            got = to_f32(y)
            for r in range(rows):
                assert oracle.compare(got[r], yref[r], 2.0 ** -8) <= BF16_DENSE_BAR, (in_f, rows, r)


def test_config4_routed_prefill_widths_mixed_rates(oracle, t3):
    # config 4's widths and rates (7168 / 2048, gate|up K2, down K3, top-8, clamp 7, bf16) with 64 rows an expert as
    # there (2048 tokens x 8 / 256), on a quarter of its experts and tokens so the CPU side stays small
    experts, hidden, inter, topk, tokens, limit = 64, 7168, 2048, 8, 512, 7
    rng = np.random.default_rng(0xC4)
    bank = oracle.synth_bank(rng, experts, hidden, inter, 32, 48)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, MCG, 0xFFFF)
    x_dev, x_f32 = make_x(rng, tokens, hidden, torch.bfloat16)
    slots, scores = routing_softmax(rng, tokens, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    y = t3.moe_clamped(x_dev.reshape(1, tokens, hidden), dbank, d_slots.reshape(1, tokens, topk),
                       d_scores.reshape(1, tokens, topk), t3.Decode.mcg, limit)
    got = to_f32(y).reshape(tokens, hidden)
    for r in (0, 300, tokens - 1):
        e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r], float(limit)))
        assert e <= BF16_MOE_BAR, f"row {r}: {e:.3e}"
    y17 = t3.moe_clamped(x_dev[:17].reshape(1, 17, hidden), dbank, d_slots[:17].reshape(1, 17, topk),
                         d_scores[:17].reshape(1, 17, topk), t3.Decode.mcg, limit)
    assert bytes_of(y17[0]) == bytes_of(y[0, :17]), "rows 0-16 of 512 tokens differ from the 17-row call"


def test_config4_routed_prefill_full_size(oracle, t3):
    # config 4 as the benchmark runs it: 2048 tokens x 256 experts, top-8, 7168 / 2048, gate|up K2, down K3, bf16, clamp 7
    # (a 3.3 GB bank, 16,384 routed positions, 96-row items). Sampled rows against ref.moeRowClamped (the reference samples
    # rows the same way, src/core/prefill_test.zig:177-182), the first 17 rows' bytes against the 17-row call, and the
    # route's integer work (rows an expert, items, placement) recounted on the host from the ids, to the bit.
    experts, hidden, inter, topk, tokens, limit = 256, 7168, 2048, 8, 2048, 7
    rng = np.random.default_rng(0xC4F)
    bank = oracle.synth_bank(rng, experts, hidden, inter, 32, 48)
    dbank = dev_bank(t3, bank)
    x_dev, x_f32 = make_x(rng, tokens, hidden, torch.bfloat16)
    slots, scores = routing_softmax(rng, tokens, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    args = (x_dev.reshape(1, tokens, hidden), dbank, d_slots.reshape(1, tokens, topk))
    plan = t3.moe_plan(*args)
    assert (plan["path"], plan["item_rows"], plan["row_slots"]) == (3, 96, tokens * topk)
    y = t3.moe_clamped(*args, d_scores.reshape(1, tokens, topk), t3.Decode.mcg, limit)
    torch.cuda.synchronize()

    # the route, read back from the workspace the call ran in
    ws = t3._workspace(x_dev.device, 0)
    p = tokens * topk

    def words(at, count):
        return ws[at:at + 4 * count].view(torch.int32).cpu().numpy().view(np.uint32)

    counts = words(plan["route_counts_at"], experts + 2)
    want_counts = np.bincount(slots.ravel(), minlength=experts).astype(np.uint32)
    assert np.array_equal(counts[:experts], want_counts), "rows an expert"
    want_items, pos = [], 0
    for e in range(experts):
        c = int(want_counts[e])
        want_items += [(e, pos + i, min(96, c - i)) for i in range(0, c, 96)]
        pos += c
    assert counts[experts] == len(want_items) and counts[experts + 1] == p, "item count and positions placed"
    items = words(plan["route_items_at"], 4 * len(want_items)).reshape(-1, 4)
    assert [tuple(int(v) for v in it[:3]) for it in items] == want_items, "items: expert, first position, rows"
    order, inv = words(plan["route_order_at"], p), words(plan["route_inv_at"], p)
    assert np.array_equal(np.sort(order), np.arange(p, dtype=np.uint32)), "order is a permutation of the row-slots"
    assert np.array_equal(order[inv], np.arange(p, dtype=np.uint32)), "inv inverts order"
    starts = np.concatenate([[0], np.cumsum(want_counts)]).astype(np.int64)
    for e in (0, 1, 100, experts - 1):  # an expert's run of positions holds exactly its row-slots
        run = order[starts[e]:starts[e + 1]]
        assert (slots.ravel()[run] == e).all()

    got = to_f32(y).reshape(tokens, hidden)
    for r in (0, 1023, tokens - 1):
        ref = RefBank(oracle, bank, MCG, 0xFFFF)  # a fresh cache a row: an expert's three W_hat are 88 MB
        e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r], float(limit)))
        assert e <= BF16_MOE_BAR, f"row {r}: {e:.3e}"
    y17 = t3.moe_clamped(x_dev[:17].reshape(1, 17, hidden), dbank, d_slots[:17].reshape(1, 17, topk),
                         d_scores[:17].reshape(1, 17, topk), t3.Decode.mcg, limit)
    assert bytes_of(y17[0]) == bytes_of(y[0, :17]), "rows 0-16 of 2048 tokens differ from the 17-row call"
