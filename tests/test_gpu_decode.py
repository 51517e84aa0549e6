"""Device decoder against the CPU oracle, bit for bit: the MFMA fragment layout the kernels assume, every
codeword of both codebooks, the quad reader at every even n and every window, and W_hat
(the bars of turboexl3 src/hip_tests.zig:24-123: exhaustive, exact)."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, dev_u16, host_u16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def t3():
    import turboexl3_amd
    from turboexl3_amd import api
    return api


def test_mfma_fragment_layout(t3):
    rng = np.random.default_rng(1)
    a = rng.standard_normal((16, 32)).astype(np.float16)
    b = rng.standard_normal((32, 16)).astype(np.float16)
    d = t3.test_mfma(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()).cpu().numpy()
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.max(np.abs(d - want)) < 1e-4
    # an asymmetric probe: one nonzero in A and in B lands in exactly one D element
    a0 = np.zeros((16, 32), dtype=np.float16)
    b0 = np.zeros((32, 16), dtype=np.float16)
    a0[5, 19] = 2.0
    b0[19, 11] = 3.0
    d0 = t3.test_mfma(torch.from_numpy(a0).cuda(), torch.from_numpy(b0).cuda()).cpu().numpy()
    want0 = np.zeros((16, 16), dtype=np.float32)
    want0[5, 11] = 6.0
    assert np.array_equal(d0, want0)


def test_codebooks_exhaustive(t3, oracle):
    mcg, mul1, t = t3.test_codebooks()
    assert np.array_equal(host_u16(mcg), oracle.codebook_table(MCG))
    assert np.array_equal(host_u16(mul1), oracle.codebook_table(MUL1))
    want_t = np.array([oracle.mul1_bytesum(c) for c in range(65536)], dtype=np.uint16)
    assert np.array_equal(host_u16(t), want_t)


def test_quad_reader_every_rate_and_window(t3, oracle):
    rng = np.random.default_rng(0x7E3A)
    tiles = 64
    mcg_tab, mul1_tab = oracle.codebook_table(MCG), oracle.codebook_table(MUL1)
    checked = 0
    for n in range(16, 130, 2):
        words = rng.integers(0, 65536, (tiles, n), dtype=np.uint16)
        want = np.stack([oracle.unpack_tile(words[i], n) for i in range(tiles)])
        dw = dev_u16(words)
        for wbits in range(8, 17):
            cw, mcg, mul1 = t3.test_lane(dw, n, wbits)
            masked = want & ((1 << wbits) - 1)
            assert np.array_equal(host_u16(cw), masked), (n, wbits)
            assert np.array_equal(host_u16(mcg), mcg_tab[masked]), (n, wbits)
            assert np.array_equal(host_u16(mul1), mul1_tab[masked]), (n, wbits)
            checked += tiles
    assert checked == 57 * 9 * tiles


@pytest.mark.parametrize("codebook", [MUL1, MCG])
@pytest.mark.parametrize("n,wbits", [(16, 16), (32, 16), (36, 16), (48, 16), (64, 16), (80, 16), (86, 16), (96, 16),
                                     (128, 16), (128, 12), (64, 8)])
def test_dequant_bit_exact(t3, oracle, codebook, n, wbits):
    rng = np.random.default_rng(n * 100 + wbits)
    in_f, out_f = 256, 384
    trellis = rng.integers(0, 65536, (in_f // 16, out_f // 16, n), dtype=np.uint16)
    got = t3.dequant(dev_u16(trellis), t3.Decode(codebook, wbits))
    want = oracle.reconstruct_inner(trellis, in_f, out_f, n, codebook, (1 << wbits) - 1)
    assert np.array_equal(host_u16(got.view(torch.int16)), want)


def test_dequant_refusals(t3):
    tr = torch.zeros(16, 24, 64, dtype=torch.int16, device="cuda")
    with pytest.raises(t3.T3Error) as e:
        t3.dequant(tr[:, :, :63].contiguous(), t3.Decode.mcg)
    assert e.value.name == "BadExl3Shape"
    with pytest.raises(t3.T3Error) as e:
        t3.dequant(tr, t3.Decode(MCG, 7))
    assert e.value.name == "Exl3WindowUnsupported"
    with pytest.raises(t3.T3Error) as e:
        t3.dequant(tr.to(torch.int32), t3.Decode.mcg)
    assert e.value.name == "BadExl3Dtype"


def test_narrowing_to_bf16_and_f16_against_the_oracle(t3, oracle):
    # the kernels narrow an output with the hardware's f32 -> bf16 / f16 conversions; held to the oracle's rule
    # (nearest even, a NaN stays a quiet NaN with its sign and top payload bits: src/test_support.zig:14-19) on exact ties
    # either way, the neighbours of every tie, overflow to infinity, subnormals, signed zeros, infinities and NaNs, and
    # on a million random bit patterns
    rng = np.random.default_rng(0xBF16)
    base = rng.integers(0, 1 << 16, 4096, dtype=np.uint32) << 16            # exact bf16 values
    ties = np.concatenate([base | 0x8000, (base | 0x8000) + 1, (base | 0x8000) - 1])
    special = np.array([0x00000000, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00001, 0x7F800001, 0xFF80FFFF,
                        0x7FFFFFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F7F8000, 0x7F7F7FFF, 0x00000001, 0x00008000, 0x00018000,
                        0x007FFFFF, 0x80008000, 0x3F808000, 0x3F818000, 0x477FE000, 0x477FF000, 0x33000000, 0x33800000],
                       dtype=np.uint32)
    bits = np.concatenate([ties.astype(np.uint32), special, rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32)])
    vals = torch.from_numpy(bits.view(np.int32)).cuda().view(torch.float32)
    bf, hf, back = t3.test_convert(vals)
    L = oracle.lib()
    want_bf = np.fromiter((L.t3o_f32_to_bf16(float(v)) if v == v else 0 for v in bits.view(np.float32)), dtype=np.uint16,
                          count=bits.size)
    nan = np.isnan(bits.view(np.float32))
    want_bf[nan] = ((bits[nan] >> 16) | 0x40).astype(np.uint16)              # ctypes would canonicalise a NaN argument
    assert np.array_equal(host_u16(bf), want_bf)
    got_hf = host_u16(hf)
    with np.errstate(over="ignore"):
        want_hf = bits.view(np.float32).astype(np.float16).view(np.uint16)
    assert np.array_equal(got_hf[~nan], want_hf[~nan])
    assert np.isnan(got_hf[nan].view(np.float16)).all()
    assert np.array_equal(back.cpu().numpy().view(np.uint32), host_u16(bf).astype(np.uint32) << 16)
