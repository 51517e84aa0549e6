"""The quant table's compute members on the device: `matmul` is `linear` and `swiglu` is `moe` / `moeClamped` with the
decode the weight carries (table/table.zig:196-222), byte for byte."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, bytes_of, dev_f16_bits, dev_u16, make_x

pytestmark = pytest.mark.gpu


def test_table_matmul_and_swiglu(oracle):
    from turboexl3_amd import api as t3
    from turboexl3_amd import table
    rng = np.random.default_rng(0x7AB)
    trunk = table.parse_block('{"format":"exl3","codebook":"mcg","window":12}')
    tr, suh, svh = oracle.synth_linear(rng, 512, 256, 64)
    d = (dev_u16(tr), dev_f16_bits(suh), dev_f16_bits(svh))
    w = table.load_tensor(trunk, *d, in_dim=512)
    x, _ = make_x(rng, 5, 512, torch.bfloat16)
    assert bytes_of(table.matmul(w, x)) == bytes_of(t3.linear(x, *d, t3.Decode(MCG, 12)))
    with pytest.raises(table.Refused) as e:
        table.load_tensor(trunk, d[0], d[1], None)
    assert (e.value.kind, e.value.why) == ("failed", "MissingWeight")

    bank_block = table.parse_block('{"format":"exl3","k":3,"codebook":"mul1"}')
    bank = oracle.synth_bank(rng, 8, 512, 256, 48)
    # a bank's trellis must be U16 itself (table/table.zig:171 admits no I16 there, unlike a trunk linear's)
    dev = lambda t, a, b: (dev_u16(t).view(torch.uint16), dev_f16_bits(a), dev_f16_bits(b))
    g, u, dn = dev(bank.gate_t, bank.gate_suh, bank.gate_svh), dev(bank.up_t, bank.up_suh, bank.up_svh), dev(bank.down_t, bank.down_suh, bank.down_svh)
    wg, wu, wd = table.load_bank(bank_block, *g, in_dim=512), table.load_bank(bank_block, *u), table.load_bank(bank_block, *dn)
    x3, _ = make_x(rng, 6, 512, torch.float16)
    x3 = x3.reshape(2, 3, 512)
    inds = torch.from_numpy(np.stack([rng.permutation(8)[:4] for _ in range(6)]).astype(np.int32)).cuda().reshape(2, 3, 4)
    scores = torch.rand(2, 3, 4, device="cuda") * 0.3
    tbank = t3.Bank(t3.Proj(*g), t3.Proj(*u), t3.Proj(*dn))
    assert bytes_of(table.swiglu(wg, wu, wd, x3, inds, scores)) == bytes_of(t3.moe(x3, tbank, inds, scores, t3.Decode.mul1))
    assert bytes_of(table.swiglu(wg, wu, wd, x3, inds, scores, limit=1)) == bytes_of(
        t3.moe_clamped(x3, tbank, inds, scores, t3.Decode.mul1, 1))
    with pytest.raises(table.Refused) as e:
        table.moe()
    assert e.value.kind == "unsupported"
