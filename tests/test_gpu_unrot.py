"""The un-rotated weight W_std and the plain GEMM over it, with the bars of turboexl3 src/core/gpu_test.zig:2294-2360:
every element of W_std within one step of its dtype of the f64 reference (or, where its 128 x 128 terms cancel, half a
step of its own plus 16 f32 epsilons of the terms' absolute sum, src/core/dense.zig:1957-1965), and the plain product
against the rotated chain within rel RMS 2^-7.5 and two steps of max|chain|'s binade."""
import math

import numpy as np
import pytest
import scipy.linalg
import torch

from tests.gpu_util import MCG, MUL1, dev_f16_bits, dev_u16, make_x, to_f32
from tests.test_gpu_dense import DenseCase

pytestmark = pytest.mark.gpu

UNROT_BAR_RMS = 2.0 ** -7 / math.sqrt(2.0)
UNROT_BAR_STEPS = 2.0
TERMS_EPS = 16.0


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def step_of(v, dtype):
    """The spacing of `dtype` at |v| (bf16: 8 significant bits, f16: 11)."""
    bits = 7 if dtype == torch.bfloat16 else 10
    a = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -24)))
    return 2.0 ** (e - bits)


def w_std_f64(case):
    """diag(suh) H W_hat H diag(svh) per 128 x 128 block in f64, and each element's sum of |terms|."""
    w_hat = case.oracle.reconstruct_inner(case.trellis, case.in_f, case.out_f, case.n, case.codebook,
                                          (1 << case.wbits) - 1).view(np.float16).astype(np.float64)
    w_hat = w_hat.reshape(case.in_f, case.out_f)
    h = scipy.linalg.hadamard(128).astype(np.float64)
    suh = case.suh.view(np.float16).astype(np.float64)
    svh = case.svh.view(np.float16).astype(np.float64)
    ref = np.empty_like(w_hat)
    terms = np.empty_like(w_hat)
    for bi in range(case.in_f // 128):
        for bo in range(case.out_f // 128):
            blk = w_hat[bi * 128:(bi + 1) * 128, bo * 128:(bo + 1) * 128]
            scale = np.outer(suh[bi * 128:(bi + 1) * 128], svh[bo * 128:(bo + 1) * 128]) / 128.0
            ref[bi * 128:(bi + 1) * 128, bo * 128:(bo + 1) * 128] = (h @ blk @ h) * scale
            terms[bi * 128:(bi + 1) * 128, bo * 128:(bo + 1) * 128] = np.abs(scale) * np.abs(blk).sum()
    return ref, terms


CASES = [
    (512, 256, 64, MCG, 16, torch.bfloat16),
    (512, 384, 48, MUL1, 16, torch.bfloat16),
    (256, 256, 128, MCG, 12, torch.float16),
    (1024, 512, 96, MUL1, 16, torch.float16),
]


@pytest.mark.parametrize("in_f,out_f,n,codebook,wbits,dtype", CASES)
def test_unrot_weight_elements_against_f64(oracle, t3, in_f, out_f, n, codebook, wbits, dtype):
    case = DenseCase(oracle, t3, 0x0707 + in_f + n, in_f, out_f, n, codebook, wbits)
    w, bad = t3.unrot_weight(case.d_trellis, case.d_suh, case.d_svh, case.dec, dtype)
    assert bad == 0 and w.shape == (in_f, out_f) and w.dtype == dtype
    got = to_f32(w).astype(np.float64)
    ref, terms = w_std_f64(case)
    d = np.abs(got - ref)
    ok = (d <= step_of(ref, dtype)) | (d <= 0.5 * step_of(got, dtype) + TERMS_EPS * 2.0 ** -23 * terms)
    assert ok.all(), f"{(~ok).sum()} of {ok.size} elements outside the element bar (worst {d.max():.3e})"
    # and the oracle's own W_std (format.reconstructPublic, f16) agrees with the same reference
    pub = oracle.reconstruct_public(case.trellis, case.suh, case.svh, in_f, out_f, n, codebook,
                                    (1 << wbits) - 1).view(np.float16).astype(np.float64).reshape(in_f, out_f)
    assert np.abs(pub - ref).max() <= 2.0 * step_of(np.abs(ref).max(), torch.float16)
    print(f"unrot {in_f}x{out_f} n={n} {dtype}: {(d > step_of(ref, dtype)).sum()} elements past one step of the reference")


def test_unrot_join_is_the_members_side_by_side_and_overflow_is_counted(oracle, t3):
    a = DenseCase(oracle, t3, 0x51, 256, 256, 64, MCG, 16)
    b = DenseCase(oracle, t3, 0x52, 256, 128, 48, MUL1, 16)
    wa, _ = t3.unrot_weight(a.d_trellis, a.d_suh, a.d_svh, a.dec, torch.bfloat16)
    wb, _ = t3.unrot_weight(b.d_trellis, b.d_suh, b.d_svh, b.dec, torch.bfloat16)
    joined = torch.zeros(256, 384, dtype=torch.bfloat16, device="cuda")
    t3.unrot_weight(a.d_trellis, a.d_suh, a.d_svh, a.dec, into=joined, col0=0)
    t3.unrot_weight(b.d_trellis, b.d_suh, b.d_svh, b.dec, into=joined, col0=256)
    assert torch.equal(joined[:, :256], wa) and torch.equal(joined[:, 256:], wb)
    # one product over the join = the members' own products, column for column
    x, _ = make_x(a.rng, 40, 256, torch.bfloat16)
    yj = t3.linear_unrot(x, joined)
    assert torch.equal(yj[:, :256], t3.linear_unrot(x, wa)) and torch.equal(yj[:, 256:], t3.linear_unrot(x, joined, 256, 128))
    # scales that push weights past f16's range: counted, not hidden
    big = np.full(256, 0x7BFF, dtype=np.uint16)  # 65504
    _, bad = t3.unrot_weight(a.d_trellis, dev_f16_bits(big), dev_f16_bits(big), a.dec, torch.float16)
    assert bad > 0


@pytest.mark.parametrize("in_f,out_f,n,codebook,dtype", [
    (512, 256, 64, MCG, torch.bfloat16),
    (2560, 640, 80, MUL1, torch.bfloat16),
    (1024, 512, 96, MUL1, torch.float16),
])
def test_linear_unrot_against_the_rotated_chain(oracle, t3, in_f, out_f, n, codebook, dtype):
    case = DenseCase(oracle, t3, 0x0717 + in_f, in_f, out_f, n, codebook, 16)
    w, bad = t3.unrot_weight(case.d_trellis, case.d_suh, case.d_svh, case.dec, dtype)
    assert bad == 0
    rows = 97
    x_dev, x_f32 = make_x(case.rng, rows, in_f, dtype)
    want = case.ref(x_f32).astype(np.float64)
    for r in (33, 97):
        # the plain launch, and the form that shares K out over the grid where the tiles are few (these shapes: all of them)
        for product in (t3.linear_unrot, t3.linear_unrot_parts):
            got = to_f32(product(x_dev[:r], w)).astype(np.float64)
            d = got - want[:r]
            rel = math.sqrt((d * d).sum() / (want[:r] ** 2).sum())
            assert rel <= UNROT_BAR_RMS, f"{product.__name__} rows {r}: rel rms {rel:.3e} over {UNROT_BAR_RMS:.3e}"
            assert np.abs(d).max() <= UNROT_BAR_STEPS * step_of(np.abs(want[:r]).max(), dtype)
        # the two sum K in different orders: a value may differ by a step of the dtype, no more
        a, b = to_f32(t3.linear_unrot(x_dev[:r], w)), to_f32(t3.linear_unrot_parts(x_dev[:r], w))
        assert np.abs(a - b).max() <= 2 * step_of(np.abs(want[:r]).max(), dtype)
    # decode and verify rows keep the trellis paths: the plain product refuses them
    with pytest.raises(t3.T3Error) as e:
        t3.linear_unrot(x_dev[:32], w)
    assert e.value.name == "Exl3EngineNotImplemented"
    print(f"linear_unrot {in_f}x{out_f} {dtype}: rel rms {rel:.3e} (bar {UNROT_BAR_RMS:.3e})")
