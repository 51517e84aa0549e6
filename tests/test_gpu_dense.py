"""The dense decode-row chain against format.project (the CPU oracle): the cases and bars of turboexl3
src/hip_tests.zig:287-350, widened to 32 rows.
  bars: f32 5e-3, bf16 2.5e-2 (f16 held to the bf16 bar's tighter f32 one plus its store rounding), measured as
  max |got - ref| / rms(ref) per row (ref.compare);
  invariants, byte for byte: a row alone equals the row among others, whatever the row count."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, host_u16, make_x, to_f32

pytestmark = pytest.mark.gpu

F32_BAR = 5e-3
BF16_BAR = 2.5e-2


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


class DenseCase:
    def __init__(self, oracle, t3, seed, in_f, out_f, n, codebook, wbits=16):
        rng = np.random.default_rng(seed)
        self.in_f, self.out_f, self.n, self.codebook, self.wbits = in_f, out_f, n, codebook, wbits
        self.trellis, self.suh, self.svh = oracle.synth_linear(rng, in_f, out_f, n)
        self.d_trellis, self.d_suh, self.d_svh = dev_u16(self.trellis), dev_f16_bits(self.suh), dev_f16_bits(self.svh)
        self.dec = t3.Decode(codebook, wbits)
        self.rng = rng
        self.oracle = oracle
        self._w_hat = None

    def ref(self, x_f32):
        if self._w_hat is None:
            self._w_hat = self.oracle.reconstruct_inner(self.trellis, self.in_f, self.out_f, self.n, self.codebook,
                                                        (1 << self.wbits) - 1)
        return self.oracle.project_rows(x_f32, self.trellis, self.suh, self.svh, self.in_f, self.out_f, self.n,
                                        self.codebook, (1 << self.wbits) - 1, threads=8, w_hat=self._w_hat)


CASES = [
    # (in, out, n, codebook, wbits, dtype): src/hip_tests.zig:294-304's list
    (512, 256, 64, MCG, 16, torch.float32),
    (512, 256, 64, MUL1, 16, torch.float32),
    (512, 384, 32, MCG, 16, torch.float32),
    (512, 256, 48, MUL1, 16, torch.float32),
    (512, 256, 36, MCG, 16, torch.float32),
    (512, 256, 128, MCG, 12, torch.float32),
    (2560, 640, 80, MUL1, 16, torch.bfloat16),
    (4096, 2048, 64, MCG, 16, torch.bfloat16),
    (1024, 512, 96, MUL1, 16, torch.float16),
    (512, 256, 112, MCG, 16, torch.float32),     # K7: the four-word wide reader (K6 and K8 read two words)
    (512, 256, 88, MUL1, 16, torch.float32),     # a fractional wide rate on the two-word reader
    # the shapes above are small enough for four tiles a load (at most 128 workgroups at eight); these two keep eight,
    # the benchmark shapes' partition: 66 x 2 and 34 x 4 workgroups
    (1024, 8448, 64, MCG, 16, torch.float32),
    (2048, 4352, 48, MUL1, 16, torch.bfloat16),
]


@pytest.mark.parametrize("in_f,out_f,n,codebook,wbits,dtype", CASES)
def test_dense_chain_rows_1_to_32(oracle, t3, in_f, out_f, n, codebook, wbits, dtype):
    case = DenseCase(oracle, t3, 0xDE45 + in_f + n, in_f, out_f, n, codebook, wbits)
    max_rows = 32
    x_dev, x_f32 = make_x(case.rng, max_rows, in_f, dtype)
    yref = case.ref(x_f32)
    bar = F32_BAR if dtype == torch.float32 else BF16_BAR
    worst = 0.0
    outs = {}
    for rows in (1, 2, 3, 4, 5, 7, 8, 9, 11, 16, 17, 24, 32):
        y = t3.linear_chain(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec)
        assert y.shape == (rows, out_f) and y.dtype == dtype
        got = to_f32(y)
        for r in range(rows):
            e = oracle.compare(got[r], yref[r])
            worst = max(worst, e)
            assert e <= bar, f"rows {rows} row {r}: {e:.3e} of rms over the bar {bar}"
        outs[rows] = y
    # each row alone gives the row's bytes, whatever the call's row count
    for rows in (7, 16, 32):
        y = outs[rows]
        for r in (0, rows // 2, rows - 1):
            alone = t3.linear_chain(x_dev[r:r + 1], case.d_trellis, case.d_suh, case.d_svh, case.dec)
            assert bytes_of(alone) == bytes_of(y[r:r + 1]), f"rows {rows}: row {r} differs from the row alone"
    print(f"dense {in_f}x{out_f} n={n} cb={codebook} {dtype}: worst {worst:.3e} (bar {bar})")


@pytest.mark.parametrize("in_f,out_f,n,codebook,wbits,dtype", [
    (4096, 2048, 64, MCG, 16, torch.bfloat16),   # per = 8: one launch up to 4 rows
    (4096, 1024, 48, MUL1, 16, torch.float16),   # deferred map: the block sums cross workgroups
    (2560, 640, 80, MUL1, 16, torch.float32),    # per = 40 > 16: prepare + arriving GEMV at every row count
    (512, 256, 36, MCG, 16, torch.float32),      # a K part that is not whole 128-blocks
    (1024, 512, 96, MCG, 12, torch.float16),     # wide reader, BT 4: two workgroup columns a 128-column block
    (1024, 8448, 64, MCG, 16, torch.float16),    # eight tiles a load (132 workgroups), per = 8
    (2048, 4352, 48, MUL1, 16, torch.bfloat16),  # eight tiles a load, the deferred map
])
def test_fused_launches_equal_the_chain_bytes(oracle, t3, in_f, out_f, n, codebook, wbits, dtype):
    # the served `linear` (one launch up to 4 rows, else prepare + arriving GEMV) against the three-launch chain,
    # byte for byte, twice in a row (the arrival counters must come back to zero)
    case = DenseCase(oracle, t3, 0xF00D + in_f + n, in_f, out_f, n, codebook, wbits)
    x_dev, _ = make_x(case.rng, 32, in_f, dtype)
    eight = n <= 64 and (out_f // 128) * t3.linear_plan(x_dev[:1], case.d_trellis, case.dec)["k_slices"] > 128
    assert t3.linear_plan(x_dev[:1], case.d_trellis, case.dec)["tiles_a_load"] == (8 if eight else 4)
    for rows in (1, 2, 3, 4, 5, 16, 17, 32):
        chain = t3.linear_chain(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec)
        for _ in range(2):
            fused = t3.linear(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec)
            assert bytes_of(fused) == bytes_of(chain), f"rows {rows}: the fused launch differs from the chain"


def test_dec_one_off_runs_the_chain(oracle, t3):
    case = DenseCase(oracle, t3, 3, 4096, 1024, 64, MCG)
    x_dev, _ = make_x(case.rng, 2, 4096, torch.float16)
    want = t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec)
    t3.configure(dec_one=0)
    try:
        got = t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec)
    finally:
        t3.configure()
    assert bytes_of(got) == bytes_of(want)


def test_dense_other_codebook_forms_stay_within_bar(oracle, t3):
    # the forms beside the served ones against the same reference: every weight the format's f16 value (mul1_defer off),
    # and MCG's hashed pair fed unrounded (mcg_pair on, this library's opt-in form)
    for cfg, books in (({"mcg_pair": 0, "mul1_defer": 0}, (MCG, MUL1)), ({"mcg_pair": 1}, (MCG,))):
        t3.configure(**cfg)
        try:
            for codebook in books:
                case = DenseCase(oracle, t3, 77 + codebook, 512, 256, 64, codebook)
                x_dev, x_f32 = make_x(case.rng, 5, 512, torch.float32)
                got = to_f32(t3.linear_chain(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec))
                yref = case.ref(x_f32)
                for r in range(5):
                    assert oracle.compare(got[r], yref[r]) <= F32_BAR, (cfg, codebook, r)
        finally:
            t3.configure()


def test_dense_leading_dims_and_outliers(oracle, t3):
    case = DenseCase(oracle, t3, 5, 512, 256, 64, MCG)
    x_dev, x_f32 = make_x(case.rng, 6, 512, torch.float16, outliers=True)
    y = t3.linear_chain(x_dev.reshape(2, 3, 512), case.d_trellis, case.d_suh, case.d_svh, case.dec)
    assert y.shape == (2, 3, 256)
    got = to_f32(y).reshape(6, 256)
    yref = case.ref(x_f32)
    for r in range(6):
        assert oracle.compare(got[r], yref[r], half_ulp=2.0 ** -11) <= F32_BAR


@pytest.mark.parametrize("in_f,out_f,n", [(128, 128, 64), (128, 256, 16), (256, 128, 128), (128, 384, 34), (384, 128, 96)])
def test_smallest_and_odd_shapes(oracle, t3, in_f, out_f, n):
    # the smallest admitted widths (one 128-block either side), the extreme rates, a fractional one, a width that is
    # three blocks: every path by its rows (one launch or arriving GEMV, chain, two MFMA blocks, trellis GEMM, W_hat form)
    for codebook in (MCG, MUL1):
        case = DenseCase(oracle, t3, 0x5A11 + in_f + out_f + n, in_f, out_f, n, codebook)
        x_dev, x_f32 = make_x(case.rng, 520, in_f, torch.float32)
        yref = case.ref(x_f32)
        for rows in (1, 2, 5, 17, 32, 33, 70, 520):
            got = to_f32(t3.linear(x_dev[:rows], case.d_trellis, case.d_suh, case.d_svh, case.dec))
            worst = max(oracle.compare(got[r], yref[r]) for r in range(rows))
            assert worst <= F32_BAR, f"{in_f}x{out_f} n={n} codebook {codebook} rows {rows}: {worst:.3e}"
        assert np.array_equal(host_u16(t3.dequant(case.d_trellis, case.dec)),
                              oracle.reconstruct_inner(case.trellis, in_f, out_f, n, codebook))


def test_dense_refusals(t3):
    tr = torch.zeros(32, 16, 64, dtype=torch.int16, device="cuda")
    suh = torch.ones(512, dtype=torch.float16, device="cuda")
    svh = torch.ones(256, dtype=torch.float16, device="cuda")
    x = torch.zeros(1, 512, dtype=torch.float16, device="cuda")

    def name(fn):
        with pytest.raises(t3.T3Error) as e:
            fn()
        return e.value.name

    assert name(lambda: t3.linear_chain(x[:, :384], tr, suh, svh, t3.Decode.mcg)) == "BadExl3Shape"
    assert name(lambda: t3.linear_chain(x, tr[:, :, :63].contiguous(), suh, svh, t3.Decode.mcg)) == "BadExl3Shape"
    assert name(lambda: t3.linear_chain(x, tr, suh[:500], svh, t3.Decode.mcg)) == "BadExl3Shape"
    assert name(lambda: t3.linear_chain(x, tr, suh, svh.to(torch.float32), t3.Decode.mcg)) == "BadExl3Dtype"
    assert name(lambda: t3.linear_chain(x.to(torch.int32), tr, suh, svh, t3.Decode.mcg)) == "BadExl3Dtype"
    assert name(lambda: t3.linear_chain(x, tr, suh, svh, t3.Decode(MCG, 17))) == "Exl3WindowUnsupported"
    # in = 16 * 30 is not a multiple of 128
    assert name(lambda: t3.linear_chain(x[:, :480], tr[:30].contiguous(), suh[:480], svh, t3.Decode.mcg)) == "BadExl3Shape"


def test_linear_bias_is_linear_plus_one_rounded_add(oracle, t3):
    # src/root.zig:358-376: the add is in x's dtype after linear's own output rounding
    case = DenseCase(oracle, t3, 0xB1A5, 512, 256, 64, MCG)
    for dtype, rows in ((torch.bfloat16, 3), (torch.float16, 40), (torch.float32, 1)):
        x_dev, _ = make_x(case.rng, rows, 512, dtype)
        bias = torch.from_numpy(case.rng.standard_normal(256).astype(np.float32)).cuda().to(dtype)
        y = t3.linear(x_dev, case.d_trellis, case.d_suh, case.d_svh, case.dec)
        got = t3.linear_bias(x_dev, case.d_trellis, case.d_suh, case.d_svh, bias, case.dec)
        want = (y.to(torch.float32) + bias.to(torch.float32)).to(dtype)
        assert bytes_of(got) == bytes_of(want)
    with pytest.raises(t3.T3Error) as e:
        t3.linear_bias(x_dev, case.d_trellis, case.d_suh, case.d_svh, bias[:128].contiguous(), case.dec)
    assert e.value.name == "BadExl3Shape"
    with pytest.raises(t3.T3Error) as e:
        t3.linear_bias(x_dev, case.d_trellis, case.d_suh, case.d_svh, bias.to(torch.float16), case.dec)
    assert e.value.name == "BadExl3Dtype"


def test_misaligned_arrays_are_refused(oracle, t3):
    # the kernels read 16 bytes a lane: an activation or scale array that starts off a 16-byte boundary is refused
    # before any launch
    case = DenseCase(oracle, t3, 5, 256, 256, 64, MCG, 16)
    x = torch.zeros(2 * 256 + 4, dtype=torch.float16, device="cuda")
    ok = x[:512].reshape(2, 256)
    off = x[4:516].reshape(2, 256)  # 8 bytes in
    t3.linear(ok, case.d_trellis, case.d_suh, case.d_svh, case.dec)
    with pytest.raises(t3.T3Error) as e:
        t3.linear(off, case.d_trellis, case.d_suh, case.d_svh, case.dec)
    assert e.value.name == "BadArgs"
