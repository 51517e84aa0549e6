"""Pins of the CPU oracle: known answers the reference's own tests hold, closed forms, brute force and
independent numpy formulations. Nothing here retypes the oracle's own formula to check itself: each check
comes from a second formulation (numpy float16 arithmetic, scipy's Hadamard, bit-by-bit stream reads)."""
import numpy as np
import pytest
import scipy.linalg

MUL1, MCG = 0, 1
EVEN_N = list(range(16, 130, 2))


# ---- f16 conversions against numpy's ------------------------------------------------------------------

def test_f16_to_f32_every_pattern(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.t3o_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rne_against_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0xF16)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        # every f16 value, and the midpoints between neighbours (ties) and just off them
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -24, 6.1e-5, -0.0, 0.0],
                 dtype=np.float32),
    ])
    f16 = np.arange(0, 0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((f16[:-1] + f16[1:]) / 2).astype(np.float32)
    vals = np.concatenate([vals, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)), -mids])
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.t3o_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rne(oracle):
    L = oracle.lib()
    assert L.t3o_f32_to_bf16(1.0) == 0x3F80
    # 1 + 2^-8 is a tie: rounds to even (1.0); the next f32 up rounds up
    assert L.t3o_f32_to_bf16(float(np.float32(1.0 + 2.0 ** -8))) == 0x3F80
    assert L.t3o_f32_to_bf16(float(np.nextafter(np.float32(1.0 + 2.0 ** -8), np.float32(2)))) == 0x3F81
    assert L.t3o_f32_to_bf16(float(np.float32(1.0 + 3 * 2.0 ** -8))) == 0x3F82
    assert L.t3o_f32_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0


# ---- codebooks -----------------------------------------------------------------------------------------

def test_mul1_known_answers(oracle):
    # src/core/format.zig:427-431
    assert oracle.decode_mul1(0) == 49896
    assert oracle.decode_mul1(1) == 14625
    assert oracle.decode_mul1(7) == 47511


def test_mcg_zero_codeword(oracle):
    # src/core/format.zig:441-445: f16(0x3B60) + f16(0x3B60) = 2 * 0.921875 = 1.84375 = 0x3F60
    assert oracle.decode_mcg(0) == 0x3F60


def _numpy_mcg(cw: np.ndarray) -> np.ndarray:
    mixed = (cw.astype(np.uint64) * 0xCBAC1FED) & 0xFFFFFFFF
    pair = (0x3B603B60 ^ (mixed & 0x8FFF8FFF)).astype(np.uint32)
    lo = (pair & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
    hi = (pair >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
    return (lo + hi).astype(np.float16).view(np.uint16)


def _numpy_mul1(cw: np.ndarray):
    mixed = ((cw.astype(np.uint64) * 0x83DCD12D) & 0xFFFFFFFF).astype(np.uint32)
    t = mixed.view(np.uint8).reshape(-1, 4).astype(np.uint32).sum(axis=1)
    h = (0x6400 + t).astype(np.uint16).view(np.float16).astype(np.float64)
    a = np.array([0x1EEE], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    b = np.array([0xC931], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    # the exact value needs 20 bits (see below), so f64 then one rounding to f16 is the fused result
    return (h * a + b).astype(np.float16).view(np.uint16), t


def test_codebooks_exhaustive_against_numpy(oracle):
    cw = np.arange(65536, dtype=np.uint32)
    assert np.array_equal(oracle.codebook_table(MCG), _numpy_mcg(cw))
    want, t = _numpy_mul1(cw)
    assert np.array_equal(oracle.codebook_table(MUL1), want)
    got_t = np.array([oracle.mul1_bytesum(int(c)) for c in cw], dtype=np.uint32)
    assert np.array_equal(got_t, t)
    assert t.max() <= 1020


def test_mul1_integer_mirror_identity(oracle):
    # src/core/lane.zig:244-254: byte pairs summed, then (bs * 0x10001 + 0x64000000) >> 16 is f16(1024 + t)
    for cw in (0, 1, 7, 0x1234, 0xFFFF):
        rr = (cw * 0x83DCD12D) & 0xFFFFFFFF
        bs = (rr & 0x00FF00FF) + ((rr >> 8) & 0x00FF00FF)
        hs_bits = (((bs * 0x00010001) + 0x64000000) & 0xFFFFFFFF) >> 16
        assert hs_bits == 0x6400 + oracle.mul1_bytesum(cw)


def test_mul1_affine_value_is_exact_in_20_bits():
    # (1024 + t) * A + B is a multiple of 2^-18 below 4 in magnitude: exact in f32, so one rounding to f16
    a = float(np.array([0x1EEE], dtype=np.uint16).view(np.float16)[0])
    b = float(np.array([0xC931], dtype=np.uint16).view(np.float16)[0])
    for t in range(0, 1021):
        v = (1024 + t) * a + b
        assert abs(v) < 4 and (v * 2 ** 18) == int(v * 2 ** 18)


# ---- rates, windows -------------------------------------------------------------------------------------

def test_windows_and_rates(oracle):
    L = oracle.lib()
    assert oracle.window_mask(16) == 0xFFFF and oracle.window_mask(12) == 0x0FFF
    assert oracle.window_mask(8) == 0xFF and oracle.window_mask(15) == 0x7FFF
    assert oracle.window_mask(7) == 0 and oracle.window_mask(17) == 0
    assert not L.t3o_rate_ok(15) and not L.t3o_rate_ok(130) and not L.t3o_rate_ok(49)
    for n in EVEN_N:
        assert L.t3o_rate_ok(n)
        ends = [L.t3o_bit_end(n, t) for t in range(256)]
        assert ends[255] == 16 * n
        fresh = [ends[0]] + [ends[t] - ends[t - 1] for t in range(1, 256)]
        assert sum(fresh) == 16 * n
    assert L.t3o_bit_end(64, 0) == 4
    assert L.t3o_bit_end(80, 15) == 80
    assert L.t3o_bit_end(36, 0) == 2 and L.t3o_bit_end(36, 3) == 9


# ---- tile readers -----------------------------------------------------------------------------------------

def _stream_bits(words: np.ndarray) -> np.ndarray:
    """The tile's bitstream by the format's rule, independent of the oracle: stream bit j = bit 31 - j%32 of
    little-endian u32 word j/32."""
    w32 = words.astype(np.uint32)[0::2] | (words.astype(np.uint32)[1::2] << 16)
    return np.array([(int(w32[j // 32]) >> (31 - j % 32)) & 1 for j in range(32 * w32.size)], dtype=np.uint8)


@pytest.mark.parametrize("n", EVEN_N)
def test_unpack_equals_definition_and_lane_plan(oracle, n):
    rng = np.random.default_rng(0xE7135EED + n)
    for _ in range(2):
        words = rng.integers(0, 65536, n, dtype=np.uint16)
        got = oracle.unpack_tile(words, n)
        bits = _stream_bits(words)
        total = 16 * n
        for t in range(256):
            end = ((t + 1) * n) >> 4
            cw = 0
            for i in range(16):
                cw = (cw << 1) | int(bits[(end + total - 16 + i) % total])
            assert got[t] == cw
            assert oracle.codeword_by_definition(words, n, t) == cw
        for lane in range(32):
            assert np.array_equal(oracle.lane_codewords(words, n, lane), got[8 * lane:8 * lane + 8])


@pytest.mark.parametrize("k", range(1, 9))
def test_packer_round_trip(oracle, k):
    # src/core/format.zig:494-510: window t's low K bits are symbol t
    rng = np.random.default_rng(0x5EED5EED + k)
    symbols = rng.integers(0, 1 << k, 256, dtype=np.uint16)
    words = oracle.pack_symbols(symbols, k)
    got = oracle.unpack_tile(words, 16 * k)
    assert np.array_equal(got & ((1 << k) - 1), symbols)
    # and the whole window is the last ceil(16/k) symbols concatenated (the trellis's shift register), circular
    bits = "".join(format(int(s), f"0{k}b") for s in symbols)
    for t in (0, 1, 5, 100, 255):
        end = (t + 1) * k
        window = (bits * 2)[len(bits) + end - 16: len(bits) + end]
        assert int(got[t]) == int(window, 2)


def test_tensor_core_perm(oracle):
    perm = oracle.tensor_core_perm()
    assert sorted(perm.tolist()) == list(range(256))
    assert perm[0] == 0 and perm[1] == 16 and perm[4] == 8
    # lane L of 32: rows 2(L%4)+{0,1,8,9}, columns L/4 and L/4+8
    for p in range(256):
        lane, i = divmod(p, 8)
        assert perm[p] // 16 == 2 * (lane % 4) + (0, 1, 8, 9)[i % 4]
        assert perm[p] % 16 == lane // 4 + 8 * (i // 4)


def test_decode_tile_and_reconstruct_inner_layout(oracle):
    rng = np.random.default_rng(11)
    n, in_f, out_f = 48, 32, 48
    trellis = rng.integers(0, 65536, (in_f // 16, out_f // 16, n), dtype=np.uint16)
    w = oracle.reconstruct_inner(trellis, in_f, out_f, n, MCG)
    perm = oracle.tensor_core_perm()
    table = oracle.codebook_table(MCG)
    for tk in range(in_f // 16):
        for tn in range(out_f // 16):
            cw = oracle.unpack_tile(trellis[tk, tn], n)
            tile = np.zeros(256, dtype=np.uint16)
            tile[perm] = table[cw]
            assert np.array_equal(w[tk * 16:(tk + 1) * 16, tn * 16:(tn + 1) * 16], tile.reshape(16, 16))
    # a window mask changes the value, not the stream
    w12 = oracle.reconstruct_inner(trellis, in_f, out_f, n, MCG, 0x0FFF)
    cw = oracle.unpack_tile(trellis[0, 0], n)
    tile = np.zeros(256, dtype=np.uint16)
    tile[perm] = table[cw & 0x0FFF]
    assert np.array_equal(w12[:16, :16], tile.reshape(16, 16))


# ---- Hadamard -----------------------------------------------------------------------------------------------

def test_hadamard_involution_and_sylvester(oracle):
    v = np.array([(i % 17) - 8.0 for i in range(128)], dtype=np.float32)
    w = oracle.hadamard128(oracle.hadamard128(v))
    assert np.max(np.abs(w - v)) < 1e-4
    H = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    rng = np.random.default_rng(5)
    x = rng.standard_normal(128).astype(np.float32)
    assert np.max(np.abs(oracle.hadamard128(x) - H @ x.astype(np.float64))) < 2e-6
    # entry sign rule (-1)^popcount(r & k)
    for r, k in ((0, 0), (1, 1), (3, 5), (127, 127), (64, 65)):
        assert H[r, k] * np.sqrt(128.0) == (-1) ** bin(r & k).count("1")
    # a unit vector picks a column: the scale and the sign of one entry
    e = np.zeros(128, dtype=np.float32)
    e[5] = 1.0
    col = oracle.hadamard128(e)
    assert np.allclose(col, H[:, 5], atol=1e-7)


def test_hadamard_butterfly_equivalence(oracle):
    # the kernels run seven butterfly stages then scale; the oracle's dense sum agrees within f32 rounding
    rng = np.random.default_rng(6)
    x = rng.standard_normal(128).astype(np.float32)
    v = x.copy()
    for s in range(7):
        bit = 1 << s
        idx = np.arange(128)
        p = v[idx ^ bit]
        v = np.where(idx & bit, p - v, v + p).astype(np.float32)
    v *= np.float32(0.08838834764831845)
    assert np.max(np.abs(v - oracle.hadamard128(x))) < 5e-6


# ---- the projection ---------------------------------------------------------------------------------------

def _f16v(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float64)


def test_project_vs_reconstruct_public_matvec(oracle):
    # src/core/format.zig:534-571
    rng = np.random.default_rng(0x7E57)
    in_f = out_f = 128
    n = 64
    trellis = rng.integers(0, 65536, (8, 8, n), dtype=np.uint16)
    suh = (0.5 + rng.random(in_f, dtype=np.float32)).astype(np.float16).view(np.uint16)
    svh = (0.5 + rng.random(out_f, dtype=np.float32)).astype(np.float16).view(np.uint16)
    pub = oracle.reconstruct_public(trellis, suh, svh, in_f, out_f, n, MUL1)
    x = (rng.random(in_f, dtype=np.float32) - 0.5).astype(np.float32)
    y = oracle.project(x, trellis, suh, svh, in_f, out_f, n, MUL1)
    acc = x.astype(np.float16).astype(np.float64) @ _f16v(pub)
    assert np.max(np.abs(acc)) > 0
    assert np.max(np.abs(acc - y)) <= 0.02 * np.max(np.abs(acc))


def test_reconstruct_public_is_the_w_std_identity(oracle):
    # W_std = diag(suh) H W_hat H diag(svh) in f64, then f16: the oracle's f32 path agrees to f16 rounding
    rng = np.random.default_rng(77)
    in_f, out_f, n = 256, 128, 32
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    w_hat = _f16v(oracle.reconstruct_inner(trellis, in_f, out_f, n, MCG))
    H = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    Hin = np.kron(np.eye(in_f // 128), H)
    Hout = np.kron(np.eye(out_f // 128), H)
    w_std = np.diag(_f16v(suh)) @ Hin @ w_hat @ Hout @ np.diag(_f16v(svh))
    got = _f16v(oracle.reconstruct_public(trellis, suh, svh, in_f, out_f, n, MCG))
    assert np.max(np.abs(got - w_std)) <= 1e-3 * np.max(np.abs(w_std)) + 1e-6


@pytest.mark.parametrize("codebook,n,mask", [(MCG, 64, 0xFFFF), (MUL1, 48, 0xFFFF), (MCG, 36, 0xFFFF), (MCG, 128, 0x0FFF)])
def test_project_against_f64_dequant_reference(oracle, codebook, n, mask):
    # the same projection in f64 with no intermediate rounding: differs only by the f16 rounding points
    rng = np.random.default_rng(1234 + n)
    in_f, out_f = 512, 256
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    x = rng.standard_normal(in_f).astype(np.float32)
    w_hat = _f16v(oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook, mask))
    H = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    xp = (x.astype(np.float16).astype(np.float64) * _f16v(suh)).reshape(-1, 128) @ H.T
    z = xp.reshape(-1) @ w_hat
    ref = (z.reshape(-1, 128) @ H.T).reshape(-1) * _f16v(svh)
    y = oracle.project(x, trellis, suh, svh, in_f, out_f, n, codebook, mask)
    assert oracle.compare(y, ref.astype(np.float32)) < 5e-3


def test_project_stages_compose_and_rows_match_bits(oracle):
    rng = np.random.default_rng(99)
    in_f, out_f, n = 256, 384, 80
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    x = rng.standard_normal((3, in_f)).astype(np.float32)
    for r in range(3):
        tr = oracle.prepare_input(x[r], suh)
        # prepared values are f16 values
        assert np.array_equal(tr, tr.astype(np.float16).astype(np.float32))
        inner = oracle.inner_gemv(trellis, tr, in_f, out_f, n, MUL1)
        y = oracle.finish_output(inner, svh)
        assert np.array_equal(y.view(np.uint32), oracle.project(x[r], trellis, suh, svh, in_f, out_f, n, MUL1).view(np.uint32))
    for threads in (1, 3):
        rows = oracle.project_rows(x, trellis, suh, svh, in_f, out_f, n, MUL1, threads=threads)
        for r in range(3):
            want = oracle.project(x[r], trellis, suh, svh, in_f, out_f, n, MUL1)
            assert np.array_equal(rows[r].view(np.uint32), want.view(np.uint32))


def test_inner_gemv_is_k_ascending_f32_sum(oracle):
    # a column's sum is sum_k xp[k] * W_hat[k, c] in f32, k ascending, mul then add (no fma), rounded to f16 once
    rng = np.random.default_rng(3)
    in_f, out_f, n = 128, 128, 64
    trellis, suh, _ = oracle.synth_linear(rng, in_f, out_f, n)
    xp = oracle.prepare_input(rng.standard_normal(in_f).astype(np.float32), suh)
    w = oracle.reconstruct_inner(trellis, in_f, out_f, n, MCG).view(np.float16).astype(np.float32)
    acc = np.zeros(out_f, dtype=np.float32)
    for k in range(in_f):
        acc = (acc + (xp[k] * w[k]).astype(np.float32)).astype(np.float32)
    want = acc.astype(np.float16).astype(np.float32)
    assert np.array_equal(oracle.inner_gemv(trellis, xp, in_f, out_f, n, MCG), want)


# ---- routed experts ---------------------------------------------------------------------------------------

def test_moe_row_slot_order_and_scale(oracle):
    # src/core/ref.zig:284-306
    rng = np.random.default_rng(0x5EED)
    bank = oracle.synth_bank(rng, 4, 256, 128, 64)
    x = rng.standard_normal(256).astype(np.float32)
    y, _ = oracle.moe_row(bank, x, [1, 3], [0.7, 0.3], MUL1)
    assert np.all(np.isfinite(y))
    rms = float(np.sqrt(np.mean(y.astype(np.float64) ** 2)))
    assert 1e-3 < rms < 100.0
    y2, _ = oracle.moe_row(bank, x, [3, 1], [0.3, 0.7], MUL1)
    assert oracle.compare(y2, y) < 1e-5


def test_moe_row_is_the_composition_of_projects(oracle):
    rng = np.random.default_rng(21)
    E, hidden, inter, n = 3, 128, 256, 48
    bank = oracle.synth_bank(rng, E, hidden, inter, n)
    x = rng.standard_normal(hidden).astype(np.float32)
    slots, scores = [2, 0], np.array([0.6, 0.4], dtype=np.float32)
    limit = 1.0
    y, hits = oracle.moe_row(bank, x, slots, scores, MCG, limit=limit)
    acc = np.zeros(hidden, dtype=np.float32)
    hg = hu = 0
    for e, w in zip(slots, scores):
        g = oracle.project(x, bank.gate_t[e], bank.gate_suh[e], bank.gate_svh[e], hidden, inter, n, MCG)
        u = oracle.project(x, bank.up_t[e], bank.up_suh[e], bank.up_svh[e], hidden, inter, n, MCG)
        hg += int(np.sum(g > limit))
        hu += int(np.sum(np.abs(u) > limit))
        gc = np.minimum(g, np.float32(limit))
        uc = np.clip(u, -limit, limit).astype(np.float32)
        h = ((gc / (np.float32(1) + np.exp(-gc).astype(np.float32))).astype(np.float32) * uc).astype(np.float32)
        d = oracle.project(h, bank.down_t[e], bank.down_suh[e], bank.down_svh[e], inter, hidden, n, MCG)
        acc = (acc + (w * d).astype(np.float32)).astype(np.float32)
    # numpy's exp may differ from libm's in the last place: a tolerance, not bytes
    assert oracle.compare(y, acc) < 1e-4
    assert hits == (hg, hu, 2 * inter)
    assert hg > 0 and hu > 0


def test_swiglu_clamp_rules(oracle):
    L = oracle.lib()
    # src/core/ref.zig:119-140: gate clamped from above only, up both ways; limit 0 = none; a NaN passes through
    def silu(g):
        return g / (1.0 + np.exp(-g))
    assert L.t3o_swiglu_clamped(10.0, 3.0, 7.0) == pytest.approx(silu(7.0) * 3.0, rel=1e-6)
    assert L.t3o_swiglu_clamped(-10.0, -30.0, 7.0) == pytest.approx(silu(-10.0) * -7.0, rel=1e-6)
    assert L.t3o_swiglu_clamped(10.0, 30.0, 0.0) == pytest.approx(silu(10.0) * 30.0, rel=1e-6)
    assert np.isnan(L.t3o_swiglu_clamped(float("nan"), 1.0, 7.0))
    assert np.isnan(L.t3o_swiglu_clamped(1.0, float("nan"), 7.0))
    assert L.t3o_swiglu_clamped_out(100.0, 3.0, 7.0) == pytest.approx(7.0 * 3.0, rel=1e-6)
    assert L.t3o_swiglu_clamped_out(1.0, -30.0, 7.0) == pytest.approx(silu(1.0) * -7.0, rel=1e-6)


def test_compare_measure(oracle):
    ref = np.array([3.0, -4.0], dtype=np.float32)
    got = np.array([3.5, -4.0], dtype=np.float32)
    rms = np.sqrt((9 + 16) / 2)
    assert oracle.compare(got, ref) == pytest.approx(0.5 / rms)
    assert oracle.compare(got, ref, half_ulp=2.0 ** -8) == pytest.approx((0.5 - 3 * 2.0 ** -8) / rms)


# ---- the reference's launch partitions (pins only; the HIP library owns its own) ---------------------------

def test_reference_partition_pins(oracle):
    L = oracle.lib()
    # src/hip/plan.zig:206-215
    assert L.t3o_rb_cap(5, 5) == 5 and L.t3o_rb_cap(6, 5) == 3
    assert L.t3o_rb_cap(16, 8) == 8 and L.t3o_rb_cap(11, 8) == 6
    assert L.t3o_bt_for(1) == 4 and L.t3o_bt_for(5) == 1
    assert L.t3o_ks_for(2560, 640) == 20
    # src/hip/plan.zig:366-371
    assert L.t3o_ks_gu(2560, 4) == 4 and L.t3o_ks_dn(640, 4) == 2
