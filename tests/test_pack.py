"""Pack loading: a synthetic EXL3 pack on disk (config.json + safetensors under the names the reference reads), claimed,
validated, loaded and run through the table; the device results equal the direct entry points', byte for byte."""
import json
import os

import numpy as np
import pytest
import torch

TRUNK = {"format": "exl3", "codebook": "mcg", "window": 16}
EXPERTS = {"format": "exl3", "k": 3, "codebook": "mcg"}


def write_pack(tmp, oracle, rng, clamp=None, model_type="qwen4_exp"):
    from safetensors.torch import save_file
    cfg = {"model_type": model_type, "trunk_quant": TRUNK, "expert_quant": EXPERTS,
           "text_config": {"num_experts_per_tok": 4}}
    if clamp:
        cfg["swiglu_limit"] = clamp
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    tr, suh, svh = oracle.synth_linear(rng, 512, 256, 64)
    bank = oracle.synth_bank(rng, 8, 512, 256, 48)
    u16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.uint16)
    i16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16))
    f16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.float16))
    tensors = {"model.layers.0.attn.q_proj.weight": i16(tr), "model.layers.0.attn.q_proj.scales": f16(suh),
               "model.layers.0.attn.q_proj.biases": f16(svh)}
    for proj, t, a, b in (("gate_proj", bank.gate_t, bank.gate_suh, bank.gate_svh), ("up_proj", bank.up_t, bank.up_suh, bank.up_svh),
                          ("down_proj", bank.down_t, bank.down_suh, bank.down_svh)):
        base = f"model.layers.0.mlp.experts.{proj}"
        tensors[f"{base}.trellis"], tensors[f"{base}.suh"], tensors[f"{base}.svh"] = u16(t), f16(a), f16(b)
    save_file({k: v for k, v in list(tensors.items())[:3]}, os.path.join(tmp, "model-00001-of-00002.safetensors"))
    save_file({k: v for k, v in list(tensors.items())[3:]}, os.path.join(tmp, "model-00002-of-00002.safetensors"))
    return (tr, suh, svh), bank


def test_pack_claims_validation_and_bill(oracle, tmp_path):
    from turboexl3_amd import pack, table
    rng = np.random.default_rng(3)
    write_pack(str(tmp_path), oracle, rng)
    p = pack.Pack(str(tmp_path), device="cpu")
    assert p.claims == {"trunk_quant": "by_marker", "expert_quant": "by_marker"}
    assert (p.blocks["expert_quant"].n, p.blocks["expert_quant"].codebook) == (48, 1)
    assert len(list(p.names())) == 12
    want = (512 // 16) * (256 // 16) * 64 * 2 + 512 * 2 + 256 * 2
    assert p.bill("trunk_quant", "model.layers.0.attn.q_proj") == want
    # without the matrix gate, or clamped, or on another model, the banks stay the built-in table's; the trunk is claimed
    assert pack.Pack(str(tmp_path), device="cpu", matrix_gate=False).claims == {"trunk_quant": "by_marker", "expert_quant": "no"}
    other = tmp_path / "clamped"
    other.mkdir()
    write_pack(str(other), oracle, rng, clamp=7.0)
    q = pack.Pack(str(other), device="cpu")
    assert q.claims["expert_quant"] == "no" and q.blocks["expert_quant"] is None
    with pytest.raises(table.Refused):
        q.bank("model.layers.0.mlp.experts.gate_proj")
    # a block the table cannot serve is refused by name when the pack opens
    bad = tmp_path / "bad"
    bad.mkdir()
    write_pack(str(bad), oracle, rng)
    cfg = json.load(open(bad / "config.json"))
    cfg["trunk_quant"]["window"] = 7
    json.dump(cfg, open(bad / "config.json", "w"))
    with pytest.raises(table.Refused) as e:
        pack.Pack(str(bad), device="cpu")
    assert e.value.why == "Exl3WindowUnsupported"


@pytest.mark.gpu
def test_pack_loads_and_runs(oracle, tmp_path):
    from tests.gpu_util import MCG, bytes_of, dev_f16_bits, dev_u16, make_x, to_f32
    from turboexl3_amd import api as t3
    from turboexl3_amd import pack, table
    rng = np.random.default_rng(4)
    (tr, suh, svh), bank = write_pack(str(tmp_path), oracle, rng)
    p = pack.Pack(str(tmp_path))
    w = p.linear("model.layers.0.attn.q_proj", in_dim=512)
    x, x_f32 = make_x(rng, 3, 512, torch.bfloat16)
    y = table.matmul(w, x)
    assert bytes_of(y) == bytes_of(t3.linear(x, dev_u16(tr), dev_f16_bits(suh), dev_f16_bits(svh), t3.Decode.mcg))
    # what the pack's tensors came to on the device, against format.project on the arrays the pack was written from
    ref = oracle.project_rows(x_f32, tr, suh, svh, 512, tr.shape[1] * 16, tr.shape[2], MCG, 0xFFFF)
    for r in range(3):
        assert oracle.compare(to_f32(y)[r], ref[r], 2.0 ** -8) <= 2.5e-2, r
    with pytest.raises(table.Refused) as e:
        p.linear("model.layers.0.attn.k_proj")
    assert (e.value.kind, e.value.why) == ("failed", "MissingWeight")
    g, u, d = (p.bank(f"model.layers.0.mlp.experts.{n}") for n in ("gate_proj", "up_proj", "down_proj"))
    x3 = x.reshape(1, 3, 512)
    inds = torch.tensor([[[0, 3, 5, 7], [1, 2, 3, 4], [7, 6, 5, 0]]], dtype=torch.int32, device="cuda")
    scores = torch.full((1, 3, 4), 0.25, device="cuda")
    dev = lambda t, a, b: t3.Proj(dev_u16(t), dev_f16_bits(a), dev_f16_bits(b))
    tbank = t3.Bank(dev(bank.gate_t, bank.gate_suh, bank.gate_svh), dev(bank.up_t, bank.up_suh, bank.up_svh),
                    dev(bank.down_t, bank.down_suh, bank.down_svh))
    y3 = table.swiglu(g, u, d, x3, inds, scores)
    assert bytes_of(y3) == bytes_of(t3.moe(x3, tbank, inds, scores, t3.Decode.mcg))
    for r in range(3):
        want, _ = oracle.moe_row(bank, x_f32[r], inds[0, r].cpu().numpy(), scores[0, r].cpu().numpy(), MCG, 0xFFFF, 0.0)
        assert oracle.compare(to_f32(y3)[0, r], want, 2.0 ** -8) <= 1.5e-2, r
