"""`t3_linear_static`: the decode-row projection whose scratch is the library's own device array. Through the C ABI,
against `t3_linear` on the same operands (the same kernels on the same launches: byte equality), on two calls in a row
with the second smaller than the first, so whatever the first left in the array is under the second; then the refusals,
and that the call allocates nothing (the caching allocator's and the driver's free memory do not move across it)."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, make_x, to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def operands(oracle, rng, in_f, out_f, n):
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    return trellis, suh, svh, dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)


def test_static_scratch_equals_linear_on_two_calls_in_a_row(oracle, t3):
    rng = np.random.default_rng(0x57A7)
    # first a call that fills a good part of the array (4 rows of a q|k|v-shaped matrix: prepared rows, block-sum copies,
    # eight planes), then a small one-row call over a different matrix: it must not see the first one's leftovers
    big = operands(oracle, rng, 4096, 12288, 64)
    small = operands(oracle, rng, 512, 256, 48)
    xb_dev, _ = make_x(rng, 4, 4096, torch.float16, outliers=True)
    xs_dev, xs_f32 = make_x(rng, 1, 512, torch.bfloat16)
    yb = torch.empty(4, 12288, dtype=torch.float16, device="cuda")
    ys = torch.empty(1, 256, dtype=torch.bfloat16, device="cuda")
    for _ in range(2):  # and again: the second round starts from the small call's leftovers
        t3.linear_static(xb_dev, *big[3:], t3.Decode.mcg, out=yb)
        t3.linear_static(xs_dev, *small[3:], t3.Decode.mul1, out=ys)
        torch.cuda.synchronize()
        assert bytes_of(yb) == bytes_of(t3.linear(xb_dev, *big[3:], t3.Decode.mcg)), "4 rows differ from t3_linear"
        assert bytes_of(ys) == bytes_of(t3.linear(xs_dev, *small[3:], t3.Decode.mul1)), "the smaller call differs"
    # and the smaller call against the oracle itself
    ref = oracle.project_rows(xs_f32, small[0], small[1], small[2], 512, 256, 48, MUL1, 0xFFFF)
    assert oracle.compare(to_f32(ys)[0], ref[0]) <= 2.5e-2


def test_static_scratch_rows_and_forms(oracle, t3):
    # every launch form of the decode rows (one launch, prepare + arriving GEMV, the chain, two row blocks) on one matrix
    rng = np.random.default_rng(0x57A8)
    ops = operands(oracle, rng, 1024, 1536, 64)
    x_dev, _ = make_x(rng, 32, 1024, torch.float32)
    for rows in (32, 1, 17, 2, 5):
        for dec in (t3.Decode.mcg, t3.Decode.mul1):
            y = t3.linear_static(x_dev[:rows], *ops[3:], dec)
            assert bytes_of(y) == bytes_of(t3.linear(x_dev[:rows], *ops[3:], dec)), (rows, dec)
    # the reset (what a caller runs after a call that did not reach its end) leaves a working array behind
    t3.linear_static_reset()
    y = t3.linear_static(x_dev[:3], *ops[3:], t3.Decode.mcg)
    assert bytes_of(y) == bytes_of(t3.linear(x_dev[:3], *ops[3:], t3.Decode.mcg))
    # rows 17..32 leave the GEMV under dense_rows_alone: the entry point refuses them then
    t3.configure(dense_rows_alone=1)
    try:
        with pytest.raises(t3.T3Error) as err:
            t3.linear_static(x_dev[:17], *ops[3:], t3.Decode.mcg)
        assert err.value.name == "Exl3EngineNotImplemented"
        y = t3.linear_static(x_dev[:16], *ops[3:], t3.Decode.mcg)
        assert bytes_of(y) == bytes_of(t3.linear(x_dev[:16], *ops[3:], t3.Decode.mcg))
    finally:
        t3.configure()


def test_static_scratch_refusals_and_no_allocation(oracle, t3):
    from turboexl3_amd import _lib
    rng = np.random.default_rng(0x57A9)
    ops = operands(oracle, rng, 512, 256, 64)
    x_dev, _ = make_x(rng, 40, 512, torch.float16)
    y = torch.full((40, 256), 7.0, dtype=torch.float16, device="cuda")
    with pytest.raises(t3.T3Error) as err:  # above the decode rows
        t3.linear_static(x_dev, *ops[3:], t3.Decode.mcg, out=y)
    assert err.value.name == "Exl3EngineNotImplemented"
    assert (y == 7.0).all().item(), "a refusal wrote to y"
    # a call whose scratch passes the array's size: 32 rows of a wide matrix (planes alone: 32 x 151936 x 4 bytes)
    wide_t = torch.zeros(128 // 16, 151936 // 16, 32, dtype=torch.int16, device="cuda")
    wide_su = torch.ones(128, dtype=torch.float16, device="cuda")
    wide_sv = torch.ones(151936, dtype=torch.float16, device="cuda")
    xw = torch.zeros(32, 128, dtype=torch.float16, device="cuda")
    need = C.c_size_t(0)
    ax, at = t3._arr(xw), t3._arr(wide_t)
    assert _lib.lib().t3_linear_workspace_bytes(C.byref(ax), C.byref(at), t3.Decode.mcg.c(), C.byref(need)) == 0
    assert need.value > _lib.STATIC_SCRATCH_BYTES
    with pytest.raises(t3.T3Error) as err:
        t3.linear_static(xw, wide_t, wide_su, wide_sv, t3.Decode.mcg)
    assert err.value.name == "WorkspaceTooSmall"
    # nothing is allocated or freed by a call: the device's free memory stays where it was
    y1 = torch.empty(1, 256, dtype=torch.float16, device="cuda")
    t3.linear_static(x_dev[:1], *ops[3:], t3.Decode.mcg, out=y1)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(3):
        t3.linear_static(x_dev[:1], *ops[3:], t3.Decode.mcg, out=y1)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_reserved() == reserved0
