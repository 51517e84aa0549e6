"""The quant table's compute members on the device: `matmul` is `linear` and `swiglu` is `moe` / `moeClamped` with the
decode the weight carries (table/table.zig:196-222): byte for byte the direct entry points, and held to the CPU oracle
(format.project, ref.moeRowClamped) with that decode by the reference's bars."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, make_x, to_f32

pytestmark = pytest.mark.gpu


def test_table_matmul_and_swiglu(oracle):
    from turboexl3_amd import api as t3
    from turboexl3_amd import table
    rng = np.random.default_rng(0x7AB)
    trunk = table.parse_block('{"format":"exl3","codebook":"mcg","window":12}')
    tr, suh, svh = oracle.synth_linear(rng, 512, 256, 64)
    d = (dev_u16(tr), dev_f16_bits(suh), dev_f16_bits(svh))
    w = table.load_tensor(trunk, *d, in_dim=512)
    x, x_f32 = make_x(rng, 5, 512, torch.bfloat16)
    y = table.matmul(w, x)
    assert bytes_of(y) == bytes_of(t3.linear(x, *d, t3.Decode(MCG, 12)))
    ref = oracle.project_rows(x_f32, tr, suh, svh, 512, 256, 64, MCG, 0x0FFF)  # the block's window: 12 bits
    for r in range(5):
        assert oracle.compare(to_f32(y)[r], ref[r], 2.0 ** -8) <= 2.5e-2, r
    with pytest.raises(table.Refused) as e:
        table.load_tensor(trunk, d[0], d[1], None)
    assert (e.value.kind, e.value.why) == ("failed", "MissingWeight")

    bank_block = table.parse_block('{"format":"exl3","k":3,"codebook":"mul1"}')
    bank = oracle.synth_bank(rng, 8, 512, 256, 48)
    # a bank's trellis must be U16 itself (table/table.zig:171 admits no I16 there, unlike a trunk linear's)
    dev = lambda t, a, b: (dev_u16(t).view(torch.uint16), dev_f16_bits(a), dev_f16_bits(b))
    g, u, dn = dev(bank.gate_t, bank.gate_suh, bank.gate_svh), dev(bank.up_t, bank.up_suh, bank.up_svh), dev(bank.down_t, bank.down_suh, bank.down_svh)
    wg, wu, wd = table.load_bank(bank_block, *g, in_dim=512), table.load_bank(bank_block, *u), table.load_bank(bank_block, *dn)
    x3, x3_f32 = make_x(rng, 6, 512, torch.float16)
    x3 = x3.reshape(2, 3, 512)
    inds = torch.from_numpy(np.stack([rng.permutation(8)[:4] for _ in range(6)]).astype(np.int32)).cuda().reshape(2, 3, 4)
    scores = torch.rand(2, 3, 4, device="cuda") * 0.3
    tbank = t3.Bank(t3.Proj(*g), t3.Proj(*u), t3.Proj(*dn))
    for limit in (0, 1):
        y = table.swiglu(wg, wu, wd, x3, inds, scores, limit=limit) if limit else table.swiglu(wg, wu, wd, x3, inds, scores)
        direct = t3.moe_clamped(x3, tbank, inds, scores, t3.Decode.mul1, limit) if limit else t3.moe(x3, tbank, inds, scores, t3.Decode.mul1)
        assert bytes_of(y) == bytes_of(direct)
        got, h_inds, h_scores = to_f32(y).reshape(6, 512), inds.cpu().numpy().reshape(6, 4), scores.cpu().numpy().reshape(6, 4)
        for r in range(6):
            want, _ = oracle.moe_row(bank, x3_f32[r], h_inds[r], h_scores[r], MUL1, 0xFFFF, float(limit))
            assert oracle.compare(got[r], want, 2.0 ** -11) <= 5e-3, (limit, r)
    with pytest.raises(table.Refused) as e:
        table.moe()
    assert e.value.kind == "unsupported"
