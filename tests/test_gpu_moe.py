"""The routed-expert decode chain against ref.moeRowClamped (the CPU oracle): the cases and bars of turboexl3
src/hip_tests.zig:444-504,885-928 (f32 5e-3, bf16 1.5e-2 of rms per row; a row alone == the row among others, byte for
byte; the four-launch form == the five-launch form, byte for byte), plus the clamp, skipped slots, mixed rates and the
shared expert."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, make_x, to_f32

pytestmark = pytest.mark.gpu

F32_BAR = 5e-3
BF16_BAR = 1.5e-2


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def dev_bank(t3, b):
    def proj(t, suh, svh):
        return t3.Proj(dev_u16(t), dev_f16_bits(suh), dev_f16_bits(svh))
    return t3.Bank(proj(b.gate_t, b.gate_suh, b.gate_svh), proj(b.up_t, b.up_suh, b.up_svh),
                   proj(b.down_t, b.down_suh, b.down_svh))


class RefBank:
    """ref.moeRowClamped composed from the oracle's `project` stages on W_hat decoded once per expert (the bits of
    format.project; tests/test_oracle_pins.py holds the composition to the C moe_row)."""

    def __init__(self, oracle, bank, codebook, mask):
        self.o, self.b, self.cb, self.mask = oracle, bank, codebook, mask
        self.cache = {}

    def _what(self, which, e):
        key = (which, e)
        if key not in self.cache:
            b = self.b
            t, in_f, out_f, n = {"gate": (b.gate_t, b.hidden, b.inter, b.n_gu), "up": (b.up_t, b.hidden, b.inter, b.n_gu),
                                 "down": (b.down_t, b.inter, b.hidden, b.n_dn)}[which]
            self.cache[key] = self.o.reconstruct_inner(t[e], in_f, out_f, n, self.cb, self.mask)
        return self.cache[key]

    def project(self, which, e, x):
        b = self.b
        t, suh, svh, in_f, out_f, n = {
            "gate": (b.gate_t, b.gate_suh, b.gate_svh, b.hidden, b.inter, b.n_gu),
            "up": (b.up_t, b.up_suh, b.up_svh, b.hidden, b.inter, b.n_gu),
            "down": (b.down_t, b.down_suh, b.down_svh, b.inter, b.hidden, b.n_dn)}[which]
        return self.o.project_rows(x[None, :], t[e], suh[e], svh[e], in_f, out_f, n, self.cb, self.mask, threads=8,
                                   w_hat=self._what(which, e))[0]

    def slot(self, e, x, limit):
        g, u = self.project("gate", e, x), self.project("up", e, x)
        if limit > 0:
            g = np.minimum(g, np.float32(limit))
            u = np.clip(u, -limit, limit).astype(np.float32)
        h = ((g / (np.float32(1) + np.exp(-g).astype(np.float32))).astype(np.float32) * u).astype(np.float32)
        return self.project("down", e, h)

    def row(self, x, slots, scores, limit=0.0):
        acc = np.zeros(self.b.hidden, dtype=np.float32)
        for e, w in zip(slots, scores):
            if 0 <= e < self.b.experts:
                acc = (acc + (np.float32(w) * self.slot(int(e), x, limit)).astype(np.float32)).astype(np.float32)
        return acc


def routing(rng, rows, topk, experts):
    slots = np.stack([rng.permutation(experts)[:topk] for _ in range(rows)]).astype(np.int32)
    scores = (0.05 + rng.random((rows, topk)) * 0.2).astype(np.float32)
    return slots, scores


CASES = [
    # (hidden, inter, experts, topk, n, codebook, wbits, dtype): src/hip_tests.zig:451-458's list
    (512, 256, 12, 4, 64, MCG, 16, torch.float32),
    (512, 256, 12, 4, 64, MUL1, 16, torch.float32),
    (512, 256, 12, 8, 36, MCG, 16, torch.float32),
    (512, 384, 12, 4, 128, MUL1, 12, torch.float32),
    (2560, 640, 16, 10, 48, MUL1, 16, torch.bfloat16),
]


@pytest.mark.parametrize("hidden,inter,experts,topk,n,codebook,wbits,dtype", CASES)
def test_moe_decode_rows_1_to_16(oracle, t3, hidden, inter, experts, topk, n, codebook, wbits, dtype):
    rng = np.random.default_rng(0xF03 + hidden + n)
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, codebook, (1 << wbits) - 1)
    dec = t3.Decode(codebook, wbits)
    max_rows = 16
    x_dev, x_f32 = make_x(rng, max_rows, hidden, dtype)
    slots, scores = routing(rng, max_rows, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    yref = np.stack([ref.row(x_f32[r], slots[r], scores[r]) for r in range(max_rows)])
    bar = F32_BAR if dtype == torch.float32 else BF16_BAR
    worst = 0.0
    for rows in (1, 2, 3, 4, 5, 8, 16):
        y = t3.moe(x_dev[:rows].reshape(1, rows, hidden), dbank, d_slots[:rows].reshape(1, rows, topk),
                   d_scores[:rows].reshape(1, rows, topk), dec)
        assert y.shape == (1, rows, hidden) and y.dtype == dtype
        got = to_f32(y).reshape(rows, hidden)
        for r in range(rows):
            e = oracle.compare(got[r], yref[r])
            worst = max(worst, e)
            assert e <= bar, f"rows {rows} row {r}: {e:.3e} over the bar {bar}"
        if rows > 1:
            for r in (0, rows - 1):
                alone = t3.moe(x_dev[r:r + 1].reshape(1, 1, hidden), dbank, d_slots[r:r + 1].reshape(1, 1, topk),
                               d_scores[r:r + 1].reshape(1, 1, topk), dec)
                assert bytes_of(alone) == bytes_of(y[0, r]), f"rows {rows}: row {r} differs from the row alone"
    print(f"moe decode {hidden}x{inter} n={n} cb={codebook} {dtype}: worst {worst:.3e} (bar {bar})")


def test_launch_forms_give_the_same_bytes(oracle, t3):
    # src/hip_tests.zig:885-928: form 9's bytes are form 3's. Here: two launches (default), four, five; twice in a
    # row (the arrival counters go back to zero), with skipped slots, a clamp and a shared expert in
    # the same launches
    rng = np.random.default_rng(9)
    # up to four rows the two-launch form runs the mid stage inside the down launch
    for codebook, n, rows, topk in ((MCG, 64, 5, 4), (MUL1, 48, 16, 4), (MUL1, 96, 3, 2), (MCG, 48, 1, 4), (MUL1, 64, 2, 3), (MCG, 64, 4, 3),
                                    (MUL1, 96, 1, 2)):
        bank = oracle.synth_bank(rng, 8, 512, 256, n)
        shared = oracle.synth_bank(rng, 1, 512, 256, n)
        dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
        x_dev, _ = make_x(rng, rows, 512, torch.bfloat16)
        slots, scores = routing(rng, rows, topk, 8)
        slots[0, 1] = -1
        slots[rows - 1, 0] = 8
        d_slots = torch.from_numpy(slots).cuda().reshape(1, rows, topk)
        d_scores = torch.from_numpy(scores).cuda().reshape(1, rows, topk)
        dec = t3.Decode(codebook, 16)
        calls = (lambda: t3.moe(x_dev.reshape(1, rows, 512), dbank, d_slots, d_scores, dec),
                 lambda: t3.moe_shared_expert(x_dev.reshape(1, rows, 512), dbank, d_slots, d_scores, dec, 1, dshared))
        for call in calls:
            nine = call()
            again = call()
            assert bytes_of(nine) == bytes_of(again)
            for form in (3, 8, 6):
                t3.configure(decode_form=form)
                try:
                    other = call()
                finally:
                    t3.configure()
                assert bytes_of(nine) == bytes_of(other), f"form 9 differs from form {form}"
    # every call left the workspace's counter area zero
    for ws in t3._workspaces.values():
        assert not ws[:65536].any()


def test_two_down_slices_in_one_workgroup_give_the_chains_bytes(oracle, t3):
    # An intermediate size of 513..1024 has two K slices of four 128-blocks in its down projection. The served launches
    # hold both in one workgroup of eight waves (five to eight of them with a block); the chains behind their own stage
    # launches keep a workgroup a slice and two planes. Same bytes: every codebook form, eight and four tiles a load (a
    # wide rate), one to sixteen rows, a skipped slot, a shared expert, and GLM's profile.
    rng = np.random.default_rng(0x2D5)
    for inter, codebook, n in ((640, MCG, 64), (1024, MUL1, 96), (896, MCG, 48), (768, MUL1, 32)):
        hidden, experts, topk = 256, 6, 3
        bank = oracle.synth_bank(rng, experts, hidden, inter, n)
        shared = oracle.synth_bank(rng, 1, hidden, inter, n)
        dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
        x_dev, x_f32 = make_x(rng, 16, hidden, torch.bfloat16)
        slots, scores = routing(rng, 16, topk, experts)
        slots[0, 1] = -1
        dec = t3.Decode(codebook, 16)
        ref = RefBank(oracle, bank, codebook, 0xFFFF)
        for rows in (1, 2, 4, 5, 16):
            d_slots = torch.from_numpy(slots[:rows]).cuda().reshape(1, rows, topk)
            d_scores = torch.from_numpy(scores[:rows]).cuda().reshape(1, rows, topk)
            x = x_dev[:rows].reshape(1, rows, hidden)
            calls = [lambda: t3.moe(x, dbank, d_slots, d_scores, dec),
                     lambda: t3.moe_shared_expert(x, dbank, d_slots, d_scores, dec, 1, dshared)]
            if rows <= 4:  # the gated shared expert rides the same launches up to four rows
                table = sigmoid_table(torch.bfloat16).cuda()
                logit = torch.from_numpy(rng.standard_normal(rows).astype(np.float32)).to(torch.bfloat16).cuda()
                calls.append(lambda: t3.moe_fused_shared(x, dbank, d_slots, d_scores, dec, dshared, table, logit))
            if codebook == MCG or n == 32:  # GLM's profile is served for MCG and for MUL1's deferred map
                k = topk + 1
                g_slots = np.concatenate([np.where(slots[:rows] < 0, 0, slots[:rows]), np.full((rows, 1), experts)], axis=1).astype(np.int32)
                dg = torch.from_numpy(g_slots).cuda().reshape(1, rows, k)
                calls.append(lambda: t3.moe_glm(x, dbank, dg, dec, 7, fill=float("nan")))
            for ci, call in enumerate(calls):
                served = call()
                assert bytes_of(served) == bytes_of(call())
                for form in (3, 6):
                    t3.configure(decode_form=form)
                    try:
                        other = call()
                    finally:
                        t3.configure()
                    assert bytes_of(served) == bytes_of(other), f"inter {inter} rows {rows} call {ci}: differs from form {form}"
            got = to_f32(calls[0]()).reshape(rows, hidden)
            for r in range(rows):
                e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r]))
                assert e <= BF16_BAR, f"inter {inter} rows {rows} row {r}: {e:.3e}"


def test_launch_forms_give_the_same_bytes_at_the_reference_rows(oracle, t3):
    # src/hip_tests.zig:891-895,907: the reference's model-sized case (2560 x 640, 16 experts, top-10, K3, MUL1's deferred
    # map, bf16) at its rows 1-5, 8 and 16
    rng = np.random.default_rng(0x909)
    hidden, inter, experts, topk = 2560, 640, 16, 10
    bank = oracle.synth_bank(rng, experts, hidden, inter, 48)
    dbank = dev_bank(t3, bank)
    x_dev, _ = make_x(rng, 16, hidden, torch.bfloat16)
    slots, scores = routing(rng, 16, topk, experts)
    dec = t3.Decode(MUL1, 16)
    for rows in (1, 2, 3, 4, 5, 8, 16):
        args = (x_dev[:rows].reshape(1, rows, hidden), dbank, torch.from_numpy(slots[:rows]).cuda().reshape(1, rows, topk),
                torch.from_numpy(scores[:rows]).cuda().reshape(1, rows, topk), dec)
        nine = t3.moe(*args)
        for form in (3, 8, 6):
            t3.configure(decode_form=form)
            try:
                other = t3.moe(*args)
            finally:
                t3.configure()
            assert bytes_of(nine) == bytes_of(other), f"rows {rows}: form 9 differs from form {form}"


@pytest.mark.parametrize("hidden,inter,experts,topk,n", [(128, 128, 1, 1, 64), (128, 256, 3, 2, 16), (384, 128, 5, 3, 128),
                                                         (256, 384, 4, 4, 34), (256, 256, 3, 2, 112), (256, 128, 3, 2, 96)])
def test_smallest_and_odd_banks(oracle, t3, hidden, inter, experts, topk, n):
    # one 128-block either side, a single expert, the extreme rates, a fractional one, three-block widths: decode rows
    # (waves past the last K part idle), the row boundary of the chains, and the prefill chain
    rng = np.random.default_rng(0xB0B + hidden + inter + n)
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    for codebook in (MCG, MUL1):
        ref = RefBank(oracle, bank, codebook, 0xFFFF)
        dec = t3.Decode(codebook, 16)
        x_dev, x_f32 = make_x(rng, 40, hidden, torch.float32)
        slots, scores = routing(rng, 40, topk, experts)
        d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
        for rows in (1, 3, 16, 17, 40):
            y = t3.moe_clamped(x_dev[:rows].reshape(1, rows, hidden), dbank, d_slots[:rows].reshape(1, rows, topk),
                               d_scores[:rows].reshape(1, rows, topk), dec, 7)
            got = to_f32(y).reshape(rows, hidden)
            for r in sorted({0, rows // 2, rows - 1}):
                e = oracle.compare(got[r], ref.row(x_f32[r], slots[r], scores[r], 7.0))
                assert e <= 5e-3, f"{hidden}/{inter} n={n} codebook {codebook} rows {rows} row {r}: {e:.3e}"


def test_clamp_skipped_slots_and_score_dtypes(oracle, t3):
    rng = np.random.default_rng(21)
    hidden, inter, experts, topk, n = 512, 256, 6, 4, 64
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    ref = RefBank(oracle, bank, MCG, 0xFFFF)
    x_dev, x_f32 = make_x(rng, 3, hidden, torch.float32)
    slots, scores = routing(rng, 3, topk, experts)
    slots[1, 2] = -1          # skipped
    slots[2, 0] = experts     # out of range: skipped
    d_slots = torch.from_numpy(slots).cuda().reshape(1, 3, topk)
    d_scores = torch.from_numpy(scores).cuda().reshape(1, 3, topk)
    x3 = x_dev.reshape(1, 3, hidden)
    limit = 1  # gate and up are O(1): a limit of 1 clamps a good share of them
    y = to_f32(t3.moe_clamped(x3, dbank, d_slots, d_scores, t3.Decode.mcg, limit)).reshape(3, hidden)
    unclamped = to_f32(t3.moe(x3, dbank, d_slots, d_scores, t3.Decode.mcg)).reshape(3, hidden)
    for r in range(3):
        want = ref.row(x_f32[r], slots[r], scores[r], float(limit))
        assert oracle.compare(y[r], want) <= F32_BAR
        assert oracle.compare(unclamped[r], ref.row(x_f32[r], slots[r], scores[r])) <= F32_BAR
        assert oracle.compare(y[r], unclamped[r]) > 0.05, "the clamp should change this case"
        _, hits = oracle.moe_row(bank, x_f32[r], slots[r], scores[r], MCG, limit=float(limit))
        assert hits[0] > 0 and hits[1] > 0
    # a limit no value reaches gives the unclamped bytes (the reference's clamped == unclamped at limit 128)
    small = oracle.synth_bank(rng, experts, hidden, inter, n)
    dsmall = dev_bank(t3, small)
    a = t3.moe_clamped(x3, dsmall, d_slots, d_scores, t3.Decode.mcg, 128)
    b = t3.moe(x3, dsmall, d_slots, d_scores, t3.Decode.mcg)
    assert bytes_of(a) == bytes_of(b)
    # scores arrive in bf16 / f16 and are widened exactly; ids as uint32
    for sdt in (torch.bfloat16, torch.float16):
        s16 = d_scores.to(sdt)
        got = t3.moe(x3, dsmall, d_slots, s16, t3.Decode.mcg)
        want = t3.moe(x3, dsmall, d_slots, s16.to(torch.float32), t3.Decode.mcg)
        assert bytes_of(got) == bytes_of(want)


def test_mixed_rates_and_shared_expert(oracle, t3):
    # gate|up at K2, down at K3 (the reference refuses mixed rates; these kernels take a rate a launch), and a shared
    # expert as one more slot of every row at weight 1
    rng = np.random.default_rng(33)
    hidden, inter, experts, topk = 512, 256, 8, 3
    bank = oracle.synth_bank(rng, experts, hidden, inter, 32, 48)
    shared = oracle.synth_bank(rng, 1, hidden, inter, 32, 48)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    ref, sref = RefBank(oracle, bank, MUL1, 0xFFFF), RefBank(oracle, shared, MUL1, 0xFFFF)
    x_dev, x_f32 = make_x(rng, 4, hidden, torch.float16)
    slots, scores = routing(rng, 4, topk, experts)
    d_slots = torch.from_numpy(slots).cuda().reshape(2, 2, topk)
    d_scores = torch.from_numpy(scores).cuda().reshape(2, 2, topk)
    x3 = x_dev.reshape(2, 2, hidden)
    half_ulp = 2.0 ** -11
    y = to_f32(t3.moe(x3, dbank, d_slots, d_scores, t3.Decode.mul1)).reshape(4, hidden)
    ys = to_f32(t3.moe_shared_expert(x3, dbank, d_slots, d_scores, t3.Decode.mul1, 0, dshared)).reshape(4, hidden)
    for r in range(4):
        routed = ref.row(x_f32[r], slots[r], scores[r])
        assert oracle.compare(y[r], routed, half_ulp) <= F32_BAR
        both = (routed + sref.slot(0, x_f32[r], 0.0)).astype(np.float32)
        assert oracle.compare(ys[r], both, half_ulp) <= F32_BAR
    # moeWithShared: the routed output rounded to x's dtype, plus a finished shared tensor, rounded again
    sh = (rng.standard_normal((2, 2, hidden)) * 0.1).astype(np.float16)
    yw = t3.moe_with_shared(x3, dbank, d_slots, d_scores, t3.Decode.mul1, False, torch.from_numpy(sh).cuda())
    want = (t3.moe(x3, dbank, d_slots, d_scores, t3.Decode.mul1).to(torch.float32) + torch.from_numpy(sh).cuda().to(torch.float32)).to(torch.float16)
    assert bytes_of(yw) == bytes_of(want)


def test_moe_refusals(oracle, t3):
    rng = np.random.default_rng(1)
    bank = oracle.synth_bank(rng, 4, 256, 128, 32)
    dbank = dev_bank(t3, bank)
    x = torch.zeros(1, 1, 256, dtype=torch.float16, device="cuda")
    inds = torch.zeros(1, 1, 2, dtype=torch.int32, device="cuda")
    scores = torch.ones(1, 1, 2, dtype=torch.float32, device="cuda")

    def name(fn):
        with pytest.raises(t3.T3Error) as e:
            fn()
        return e.value.name

    assert name(lambda: t3.moe_clamped(x, dbank, inds, scores, t3.Decode.mcg, 0)) == "InvalidExl3Clamp"
    assert name(lambda: t3.moe_clamped(x, dbank, inds, scores, t3.Decode.mcg, 129)) == "InvalidExl3Clamp"
    assert name(lambda: t3.moe(x[0], dbank, inds, scores, t3.Decode.mcg)) == "BadExl3Shape"
    assert name(lambda: t3.moe(x, dbank, inds, scores[:, :, :1], t3.Decode.mcg)) == "BadExl3Shape"
    big = torch.zeros(1, 1, 33, dtype=torch.int32, device="cuda")
    assert name(lambda: t3.moe(x, dbank, big, torch.ones(1, 1, 33, device="cuda"), t3.Decode.mcg)) == "BadExl3Shape"
    assert name(lambda: t3.moe(x, dbank, inds.to(torch.int16), scores, t3.Decode.mcg)) == "BadExl3Dtype"
    assert name(lambda: t3.moe(x, dbank, inds, scores.to(torch.int32), t3.Decode.mcg)) == "BadExl3Dtype"
    mism = oracle.synth_bank(rng, 4, 256, 128, 32)
    mism.up_t = rng.integers(0, 65536, (4, 16, 8, 48), dtype=np.uint16)
    assert name(lambda: t3.moe(x, dev_bank(t3, mism), inds, scores, t3.Decode.mcg)) == "Exl3GateUpRateMismatch"
    bad = oracle.synth_bank(rng, 4, 256, 128, 32)
    bad.down_svh = bad.down_svh[:, :128]
    assert name(lambda: t3.moe(x, dev_bank(t3, bad), inds, scores, t3.Decode.mcg)) == "BadExl3Shape"


def test_silu_out_clamp_decode_and_prefill_rows(oracle, t3):
    # Ling-3.1's clamp (format.ClampAt.silu_out; ref.moeRowClampedAt at silu_out): min(silu(g), L) * clamp(u, -L, L)
    rng = np.random.default_rng(0x51C)
    hidden, inter, experts, topk, n = 512, 256, 6, 3, 64
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    rows = 40
    x_dev, x_f32 = make_x(rng, rows, hidden, torch.float32)
    x_dev, x_f32 = x_dev * 3.0, x_f32 * np.float32(3.0)  # gates large enough that silu(g) passes the limit
    slots, scores = routing(rng, rows, topk, experts)
    d_slots, d_scores = torch.from_numpy(slots).cuda(), torch.from_numpy(scores).cuda()
    limit = 1
    for count in (3, rows):  # the decode chain, then the prefill chain
        args = (x_dev[:count].reshape(1, count, hidden), dbank, d_slots[:count].reshape(1, count, topk),
                d_scores[:count].reshape(1, count, topk), t3.Decode.mcg)
        out = to_f32(t3.moe_swiglu(*args, limit, t3.SILU_OUT)).reshape(count, hidden)
        gate_in = to_f32(t3.moe_swiglu(*args, limit, t3.GATE_IN)).reshape(count, hidden)
        assert bytes_of(t3.moe_swiglu(*args, limit, t3.GATE_IN)) == bytes_of(t3.moe_clamped(*args, limit))
        assert bytes_of(t3.moe_swiglu(*args, 0, t3.SILU_OUT)) == bytes_of(t3.moe(*args))
        for r in (0, count - 1):
            want, hits = oracle.moe_row(bank, x_f32[r], slots[r], scores[r], MCG, limit=float(limit), clamp_at=1)
            assert hits[0] > 0 and hits[1] > 0
            assert oracle.compare(out[r], want) <= F32_BAR
            assert oracle.compare(out[r], gate_in[r]) > 1e-2, "the two clamps should differ on this case"
    with pytest.raises(t3.T3Error) as e:
        t3.moe_swiglu(*args, 5, 2)
    assert e.value.name == "InvalidExl3Clamp"


def sigmoid_table(dtype):
    """The host's table: the sigmoid of every 16-bit pattern of `dtype`, in `dtype` (what MLX's Sigmoid gives the
    reference; torch's here)."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    return torch.sigmoid(bits.view(dtype).to(torch.float32)).to(dtype)


def _to(dtype, a):
    """float32 values rounded to `dtype` and back."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).to(torch.float32).numpy()


def _tab(table_f32, dtype, a):
    """table[bits of a] for values already of `dtype`."""
    bits = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).view(torch.int16).to(torch.int32) & 0xFFFF
    return table_f32[bits.numpy()]


@pytest.mark.parametrize("codebook,n,dtype", [(MCG, 64, torch.bfloat16), (MUL1, 48, torch.float16)])
def test_fused_gated_shared_expert(oracle, t3, codebook, n, dtype):
    # src/models/qwen38/api.zig:305-312: y = routed + sigmoid(logit) * shared(x) at up to 4 rows, with the roundings of
    # the host's chain (the routed sum, the table SwiGLU, the gate, the product and the add each round to the dtype)
    rng = np.random.default_rng(0x5A3 + n)
    hidden, inter, experts, topk = 512, 256, 8, 4
    bank, shared = oracle.synth_bank(rng, experts, hidden, inter, n), oracle.synth_bank(rng, 1, hidden, inter, n)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    ref, sref = RefBank(oracle, bank, codebook, 0xFFFF), RefBank(oracle, shared, codebook, 0xFFFF)
    dec = t3.Decode(codebook, 16)
    rows = 4
    x_dev, x_f32 = make_x(rng, rows, hidden, dtype)
    slots, scores = routing(rng, rows, topk, experts)
    slots[1, 2] = -1
    logit = torch.from_numpy(rng.standard_normal(rows).astype(np.float32)).to(dtype)
    table = sigmoid_table(dtype)
    table_f32 = table.to(torch.float32).numpy()
    want = []
    for r in range(rows):
        routed = _to(dtype, ref.row(x_f32[r], slots[r], scores[r]))
        gt, ut = _to(dtype, sref.project("gate", 0, x_f32[r])), _to(dtype, sref.project("up", 0, x_f32[r]))
        act = _to(dtype, gt * _tab(table_f32, dtype, gt))
        h = _to(dtype, act * ut)
        sterm = _to(dtype, sref.project("down", 0, h))
        gated = _to(dtype, _tab(table_f32, dtype, logit[r:r + 1].to(torch.float32).numpy()) * sterm)
        want.append(_to(dtype, routed + gated))
    d_slots = torch.from_numpy(slots).cuda()
    d_scores = torch.from_numpy(scores).cuda()
    first = None
    # bf16: the output passes three roundings of the dtype at the end (the routed sum, the gated product, the add) where
    # `moe` has one, and a step of bf16 at 4 rms is 3e-2 of rms: the dense bar (src/hip_tests.zig:326), not the routed
    # one. f16: two steps of f16 at 4 rms (8e-3 of rms) on top of the f32 bar's share
    bar = 2.5e-2 if dtype == torch.bfloat16 else 1e-2
    for form in (9, 8, 3, 6, 5, 7):
        t3.configure(decode_form=form)
        try:
            for count in (1, 3, 4):
                y = t3.moe_fused_shared(x_dev[:count].reshape(1, count, hidden), dbank,
                                        d_slots[:count].reshape(1, count, topk), d_scores[:count].reshape(1, count, topk),
                                        dec, dshared, table.cuda(), logit[:count].cuda())
                got = to_f32(y).reshape(count, hidden)
                for r in range(count):
                    e = oracle.compare(got[r], want[r])
                    assert e <= bar, f"form {form} rows {count} row {r}: {e:.3e} over the bar {bar}"
                if count == 4:
                    if first is None:
                        first = bytes_of(y)
                    else:
                        assert bytes_of(y) == first, f"form {form}: other bytes than the two-launch form"
        finally:
            t3.configure()
    # beyond the shared rows the fused launches refuse, and so does an f32 call: the caller keeps its chain
    x5, _ = make_x(rng, 5, hidden, dtype)
    s5, w5 = routing(rng, 5, topk, experts)
    with pytest.raises(t3.T3Error) as err:
        t3.moe_fused_shared(x5.reshape(1, 5, hidden), dbank, torch.from_numpy(s5).cuda().reshape(1, 5, topk),
                            torch.from_numpy(w5).cuda().reshape(1, 5, topk), dec, dshared, table.cuda(),
                            torch.zeros(5, dtype=dtype, device="cuda"))
    assert err.value.name == "Exl3EngineNotImplemented"


def router_reference(logits_f32, k, dtype):
    """The host's softmax router as src/models/qwen38/kernels/shared/router_softmax_*.metal restates it: top-k by logit
    (ties to the lowest id), weights = dtype(softmax over all experts), renormalised by their total added up in slot
    order in the dtype."""
    rows = logits_f32.shape[0]
    inds = np.zeros((rows, k), dtype=np.int32)
    scores = np.zeros((rows, k), dtype=np.float32)
    for r in range(rows):
        row = logits_f32[r]
        pick = np.argsort(-row, kind="stable")[:k]
        smax = row.max()
        snorm = np.float32(1.0) / np.exp(row - smax, dtype=np.float32).sum(dtype=np.float32)
        w = _to(dtype, np.exp(row[pick] - smax, dtype=np.float32) * snorm)
        tot = np.float32(0.0)
        for j in range(k):
            tot = _to(dtype, np.array([w[j] + tot]))[0]
        inds[r] = pick
        scores[r] = _to(dtype, w / tot)
    return inds, scores


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_gated_shared_expert_with_the_router_inside(oracle, t3, dtype):
    # src/models/qwen38/api.zig:386-395: the same call with the top-k and the renormalised softmax weights made from the
    # router's logits by one launch in front
    rng = np.random.default_rng(0x5A7)
    hidden, inter, experts, k, n = 512, 256, 70, 6, 64
    bank, shared = oracle.synth_bank(rng, experts, hidden, inter, n), oracle.synth_bank(rng, 1, hidden, inter, n)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    dec = t3.Decode(MCG, 16)
    rows = 3
    x_dev, _ = make_x(rng, rows, hidden, dtype)
    logits = torch.from_numpy(rng.standard_normal((rows, experts)).astype(np.float32)).to(dtype)
    logits[1, 5] = logits[1, 40] = 9.0  # a tie at the top: the lowest id first
    logit = torch.from_numpy(rng.standard_normal(rows).astype(np.float32)).to(dtype)
    table = sigmoid_table(dtype).cuda()
    y, inds, scores = t3.moe_fused_shared_routed(x_dev.reshape(1, rows, hidden), dbank, logits.cuda().reshape(1, rows, experts),
                                                 k, dec, dshared, table, logit.cuda(), return_routing=True)
    want_i, want_s = router_reference(logits.to(torch.float32).numpy(), k, dtype)
    assert np.array_equal(inds.cpu().numpy(), want_i), "the router picked other experts"
    assert want_i[1, 0] == 5 and want_i[1, 1] == 40
    step = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert np.abs(to_f32(scores) - want_s).max() <= step * want_s.max() * 2, "weights further than a step of the dtype"
    # and the call is the unrouted one on the router's own slots and weights, byte for byte
    same = t3.moe_fused_shared(x_dev.reshape(1, rows, hidden), dbank, inds.reshape(1, rows, k), scores.reshape(1, rows, k),
                               dec, dshared, table, logit.cuda())
    assert bytes_of(y) == bytes_of(same)
    with pytest.raises(t3.T3Error) as err:  # more experts a token than the router carries
        t3.moe_fused_shared_routed(x_dev.reshape(1, rows, hidden), dbank, logits.cuda().reshape(1, rows, experts), 32, dec,
                                   dshared, table, logit.cuda())
    assert err.value.name == "Exl3EngineNotImplemented"


def gate_logit_reference(x, gv):
    """x [rows, D], gv [D] (bf16 values in f32) -> bf16 logits, summed as src/core/kernels/sources/gate_gemv.metal and
    gate_sum.metal state MLX's gemv: lane t of 256 adds columns 4 t + 1024 i + tn in order, each group of 32 lanes folds
    a shuffle-down tree, the 8 partials are added in order. Every operation in f32."""
    rows, d = x.shape
    out = np.zeros(rows, dtype=np.float32)
    for r in range(rows):
        res = np.zeros(256, dtype=np.float32)
        for i in range(0, d, 1024):
            for tn in range(4):
                c = 4 * np.arange(256) + i + tn
                ok = c < d
                prod = np.zeros(256, dtype=np.float32)
                prod[ok] = x[r, c[ok]] * gv[c[ok]]
                res = (res + prod).astype(np.float32)
        v = res.reshape(8, 32).copy()
        for off in (16, 8, 4, 2, 1):
            nxt = v.copy()
            nxt[:, :32 - off] = v[:, :32 - off] + v[:, off:]
            v = nxt
        total = v[0, 0]
        for g in range(1, 8):
            total = np.float32(total + v[g, 0])
        out[r] = total
    return torch.from_numpy(out).to(torch.bfloat16)


@pytest.mark.parametrize("hidden,rows", [(512, 2), (2560, 3), (2048, 4)])
def test_fused_gated_shared_expert_with_the_gate_vector(oracle, t3, hidden, rows):
    # src/models/qwen38/api.zig:386-416: with the shared gate's weight vector in the logit's place the router's launch
    # also takes each row's logit, in the order the reference states for MLX's gemv. That order is a fixed sequence of f32
    # operations (a product of two bf16 values is exact in f32), so the logits are held to their bytes against a numpy
    # statement of it, which in turn sits within a bf16 step of the float64 dot; the call then equals the one given
    # those logits, byte for byte.
    rng = np.random.default_rng(0x6A7E + hidden)
    inter, experts, k, n = 256, 12, 4, 48
    bank, shared = oracle.synth_bank(rng, experts, hidden, inter, n), oracle.synth_bank(rng, 1, hidden, inter, n)
    dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
    dec = t3.Decode(MCG, 16)
    dtype = torch.bfloat16
    x_dev, x_f32 = make_x(rng, rows, hidden, dtype)
    logits = torch.from_numpy(rng.standard_normal((rows, experts)).astype(np.float32)).to(dtype).cuda()
    gv = torch.from_numpy((rng.standard_normal(hidden) * 0.05).astype(np.float32)).to(dtype)
    table = sigmoid_table(dtype).cuda()
    x3, l3 = x_dev.reshape(1, rows, hidden), logits.reshape(1, rows, experts)
    y, inds, scores, glogit = t3.moe_fused_shared_routed(x3, dbank, l3, k, dec, dshared, table, None, return_routing=True,
                                                         gate_vec=gv.cuda())
    want = gate_logit_reference(x_f32, gv.to(torch.float32).numpy())
    assert bytes_of(glogit.cpu()) == bytes_of(want), "the gate's logits differ from the stated order's"
    exact = x_f32.astype(np.float64) @ gv.to(torch.float64).numpy()
    assert np.all(np.abs(want.to(torch.float64).numpy() - exact) <= 2.0 ** -8 * np.maximum(np.abs(exact), 2.0 ** -6))
    same = t3.moe_fused_shared_routed(x3, dbank, l3, k, dec, dshared, table, glogit)
    assert bytes_of(y) == bytes_of(same)
    for kwargs, logit, xs, name in (
        ({"gate_vec": gv.cuda()}, glogit, x3, "BadExl3Shape"),                     # both
        ({}, None, x3, "BadExl3Shape"),                                             # neither
        ({"gate_vec": gv.cuda()}, None, x3[:, :1], "Exl3EngineNotImplemented"),     # one row: not that gemv
        ({"gate_vec": gv[:hidden - 128].contiguous().cuda()}, None, x3, "Exl3EngineNotImplemented"),
        ({"gate_vec": gv.to(torch.float16).cuda()}, None, x3, "Exl3EngineNotImplemented"),
    ):
        with pytest.raises(t3.T3Error) as err:
            t3.moe_fused_shared_routed(xs, dbank, l3[:, :xs.shape[1]], k, dec, dshared, table, logit, **kwargs)
        assert err.value.name == name, (kwargs.keys(), name)


def test_grouped_form_serves_an_experts_row_slots_together(oracle, t3):
    """The six-launch form (the row-slots that read one expert served by one set of workgroups, up to sixteen a group):
    the bytes of the five launches, where every row reads the same experts (full groups), where a row names an expert
    twice (more than sixteen readers: a second group), with skipped ids and a shared expert (one group of every row), at
    four tiles a load as well; and where the default configuration picks it by itself (large experts, several rows)."""
    rng = np.random.default_rng(0x6E0)
    hidden, inter = 512, 256
    for experts, topk, n, rows, how in ((2, 2, 64, 16, "same"), (3, 2, 48, 16, "twice"), (12, 4, 80, 9, "mixed"),
                                        (5, 3, 96, 2, "mixed")):
        bank = oracle.synth_bank(rng, experts, hidden, inter, n)
        shared = oracle.synth_bank(rng, 1, hidden, inter, n)
        dbank, dshared = dev_bank(t3, bank), dev_bank(t3, shared)
        x_dev, _ = make_x(rng, rows, hidden, torch.bfloat16)
        slots, scores = routing(rng, rows, topk, experts)
        if how == "same":
            slots[:] = np.arange(topk, dtype=np.int32)[None, :]
        elif how == "twice":
            slots[:] = 1                                   # expert 1 read 32 times: two groups of sixteen
        else:
            slots[0, 1] = -1
            slots[rows - 1, 0] = experts + 3
        args = (x_dev.reshape(1, rows, hidden), dbank, torch.from_numpy(slots).cuda().reshape(1, rows, topk),
                torch.from_numpy(scores).cuda().reshape(1, rows, topk), t3.Decode(MUL1 if n == 48 else MCG, 16))
        for call in (lambda: t3.moe_clamped(*args, 7), lambda: t3.moe_shared_expert(*args, 1, dshared)):
            t3.configure(decode_form=3)
            try:
                five = call()
            finally:
                t3.configure()
            t3.configure(decode_form=6)
            try:
                six, again = call(), call()
            finally:
                t3.configure()
            assert bytes_of(six) == bytes_of(five), f"{how} E {experts} top-{topk} n {n} rows {rows}: grouped differs"
            assert bytes_of(six) == bytes_of(again)
    # the default's own choice: 4096 x 2048, sixteen rows over few experts
    hidden, inter, experts, topk = 4096, 2048, 4, 3
    bank = dev_bank(t3, oracle.synth_bank(rng, experts, hidden, inter, 64))
    x_dev, _ = make_x(rng, 16, hidden, torch.bfloat16)
    slots, scores = routing(rng, 16, topk, experts)
    args = (x_dev.reshape(1, 16, hidden), bank, torch.from_numpy(slots).cuda().reshape(1, 16, topk),
            torch.from_numpy(scores).cuda().reshape(1, 16, topk), t3.Decode.mcg)
    assert t3.moe_plan(args[0], bank, args[2])["launches"] == 6
    served = t3.moe(*args)
    t3.configure(decode_form=3)
    try:
        five = t3.moe(*args)
    finally:
        t3.configure()
    assert bytes_of(served) == bytes_of(five)


def test_glm_profile_launch_forms_give_the_same_bytes(oracle, t3):
    # src/hip_tests.zig:896,900-913: form 9's bytes are form 3's under GLM's profile too (4096 x 2048, 9 experts, K4, MCG,
    # bf16, the last slot of a row the host's shared expert), rows 1-5, 8 and 16; and with MUL1's deferred map
    rng = np.random.default_rng(0x90A)
    for hidden, inter, experts, n, codebook in ((4096, 2048, 9, 64, MCG), (512, 384, 6, 48, MUL1)):
        topk = min(8, experts - 1)
        k = topk + 1
        bank = oracle.synth_bank(rng, experts, hidden, inter, n)
        dbank = dev_bank(t3, bank)
        x_dev, _ = make_x(rng, 16, hidden, torch.bfloat16)
        slots = np.stack([np.concatenate([rng.permutation(experts)[:topk], [experts]]) for _ in range(16)]).astype(np.int32)
        for rows in (1, 2, 3, 4, 5, 8, 16):
            args = (x_dev[:rows].reshape(1, rows, hidden), dbank, torch.from_numpy(slots[:rows]).cuda().reshape(1, rows, k),
                    t3.Decode(codebook, 16), 7)
            two = t3.moe_glm(*args, fill=float("nan"))
            again = t3.moe_glm(*args, fill=float("nan"))
            assert bytes_of(two) == bytes_of(again)
            for form in (3, 6):
                t3.configure(decode_form=form)
                try:
                    five = t3.moe_glm(*args, fill=float("nan"))
                finally:
                    t3.configure()
                assert bytes_of(two) == bytes_of(five), f"hidden {hidden} rows {rows}: the served form differs from form {form}"
            assert torch.isnan(two.reshape(rows, k, hidden)[:, topk]).all(), "the slot past the experts was written"


def _bf16_round64(v):
    return torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


def _w_std64(oracle, trellis, suh, svh, in_f, out_f, n, codebook):
    """diag(suh) H W_hat H diag(svh) in f64 (src/hip_tests.zig:546-554 dequant64)."""
    import scipy.linalg
    w = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook, 0xFFFF).view(np.float16).astype(np.float64).reshape(in_f, out_f)
    h = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    w = (h @ w.reshape(in_f // 128, 128, out_f)).reshape(in_f, out_f)          # rotate the input side, block by block
    w = w * suh.view(np.float16).astype(np.float64)[:, None]
    w = (w.reshape(in_f, out_f // 128, 128) @ h).reshape(in_f, out_f)           # and the output side
    return w * svh.view(np.float16).astype(np.float64)[None, :]


@pytest.mark.parametrize("hidden,inter,experts,rows", [(512, 256, 12, 1), (512, 256, 12, 4), (512, 256, 12, 8),
                                                        (512, 256, 12, 40), (4096, 2048, 9, 8), (4096, 2048, 9, 40)])
def test_glm_profile_slots_against_float64(oracle, t3, hidden, inter, experts, rows):
    # src/hip_tests.zig:576-671,762-797 (both of its shapes): every routed slot's f32 output within
    # sum |a w| / 64 + 1e-6 of float64 under GLM's roundings, the slot past the experts (the host's shared expert) left
    # alone; 40 rows take the prefill chain, where the reference samples rows 0, 1, 20 and 39
    rng = np.random.default_rng(0x61A)
    topk, n, limit = 8, 64, 7.0
    bank = oracle.synth_bank(rng, experts, hidden, inter, n)
    dbank = dev_bank(t3, bank)
    k = topk + 1
    x_dev, x_f32 = make_x(rng, rows, hidden, torch.bfloat16)
    slots = np.stack([np.concatenate([rng.permutation(experts)[:topk], [experts]]) for _ in range(rows)]).astype(np.int32)
    y = t3.moe_glm(x_dev.reshape(1, rows, hidden), dbank, torch.from_numpy(slots).cuda().reshape(1, rows, k),
                   t3.Decode(MCG, 16), int(limit), fill=float("nan"))
    got = y.cpu().numpy().reshape(rows, k, hidden).astype(np.float64)
    assert np.isnan(got[:, topk]).all(), "the slot past the experts was written"
    worst = 0.0
    w64 = {}
    sampled = range(rows) if rows <= 8 and hidden <= 512 else sorted({0, 1, rows // 2, rows - 1})
    for r in sampled:
        xr = x_f32[r].astype(np.float64)
        for j in range(topk):
            e = int(slots[r, j])
            if e not in w64:
                w64[e] = (_w_std64(oracle, bank.gate_t[e], bank.gate_suh[e], bank.gate_svh[e], hidden, inter, n, MCG),
                          _w_std64(oracle, bank.up_t[e], bank.up_suh[e], bank.up_svh[e], hidden, inter, n, MCG),
                          _w_std64(oracle, bank.down_t[e], bank.down_suh[e], bank.down_svh[e], inter, hidden, n, MCG))
            wg, wu, wd = w64[e]
            gg, uu = _bf16_round64(xr @ wg), _bf16_round64(xr @ wu)
            gg, uu = np.minimum(gg, limit), np.clip(uu, -limit, limit)
            act = _bf16_round64(_bf16_round64(gg / (1.0 + np.exp(-gg))) * uu)
            want = act @ wd
            tol = np.abs(act[:, None] * wd).sum(axis=0) / 64.0 + 1e-6
            q = (np.abs(got[r, j] - want) / tol).max()
            assert q <= 1.0, f"rows {rows} row {r} slot {j}: {q:.3f} of its tolerance"
            worst = max(worst, q)
    print(f"GLM profile hidden {hidden} rows {rows}: worst {worst:.3f} of the float64 tolerance")
