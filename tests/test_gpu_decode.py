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
