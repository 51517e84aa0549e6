"""The committed known-answer vectors (tests/golden/exl3_golden.json, written by tests/golden/make_golden.py from the
format's definition and the reference's own test literals) against the C oracle on the CPU, and against the device
decoder on the GPU."""
import hashlib
import json
import os

import numpy as np
import pytest

MUL1, MCG = 0, 1
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "exl3_golden.json")


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def _sha(a: np.ndarray) -> str:
    return hashlib.sha256(a.astype("<u2").tobytes()).hexdigest()


def test_generator_reproduces_the_committed_file(golden, tmp_path, monkeypatch):
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(GOLDEN), "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    monkeypatch.setattr(mod, "HERE", str(tmp_path))
    mod.main()
    with open(tmp_path / "exl3_golden.json") as f:
        assert json.load(f) == golden


def test_oracle_codebooks(oracle, golden):
    for cw, want in golden["mul1_known"].items():
        assert oracle.decode_mul1(int(cw)) == want
    for cw, want in golden["mcg_known"].items():
        assert oracle.decode_mcg(int(cw)) == want
    mcg, mul1 = oracle.codebook_table(MCG), oracle.codebook_table(MUL1)
    assert _sha(mcg) == golden["mcg_table_sha256"]
    assert _sha(mul1) == golden["mul1_table_sha256"]
    for cw, want in golden["mcg_samples"].items():
        assert int(mcg[int(cw)]) == want
    for cw, want in golden["mul1_samples"].items():
        assert int(mul1[int(cw)]) == want


def test_oracle_tiles_perm_windows_partitions(oracle, golden):
    L = oracle.lib()
    for n, tile in golden["tiles"].items():
        words = np.array(tile["trellis_u16"], dtype=np.uint16)
        want = np.array(tile["codewords"], dtype=np.uint16)
        assert np.array_equal(oracle.unpack_tile(words, int(n)), want), n
        got = np.concatenate([oracle.lane_codewords(words, int(n), lane) for lane in range(32)])
        assert np.array_equal(got, want), n
    perm = oracle.tensor_core_perm()
    assert perm.tolist() == golden["tensor_core_perm"]
    for p, want in golden["perm_known"].items():
        assert int(perm[int(p)]) == want
    for bits, want in golden["window_masks"].items():
        assert oracle.window_mask(int(bits)) == want
    for n, ends in golden["bit_end"].items():
        for t, want in ends.items():
            assert ((int(t) + 1) * int(n)) >> 4 == want
    pins = golden["partition_pins"]
    for a, b, want in pins["rb_cap"]:
        assert L.t3o_rb_cap(a, b) == want
    for a, want in pins["bt_for"]:
        assert L.t3o_bt_for(a) == want
    for a, b, want in pins["ks_for"]:
        assert L.t3o_ks_for(a, b) == want
    for hidden, inter, gu, dn in pins["ks_gu_dn"]:
        assert L.t3o_ks_gu(hidden, 4) == gu and L.t3o_ks_dn(inter, 4) == dn


@pytest.mark.gpu
def test_device_decoder_against_golden(golden):
    import torch

    from tests.gpu_util import dev_u16, host_u16
    from turboexl3_amd import api as t3
    mcg, mul1, _ = t3.test_codebooks()
    mcg, mul1 = host_u16(mcg), host_u16(mul1)
    assert _sha(mcg) == golden["mcg_table_sha256"]
    assert _sha(mul1) == golden["mul1_table_sha256"]
    for n, tile in golden["tiles"].items():
        words = np.array(tile["trellis_u16"], dtype=np.uint16)[None, :]
        want = np.array(tile["codewords"], dtype=np.uint16)
        cw, dm, d1 = t3.test_lane(dev_u16(words), int(n), 16)
        assert np.array_equal(host_u16(cw)[0], want), n
        assert np.array_equal(host_u16(dm)[0], mcg[want]) and np.array_equal(host_u16(d1)[0], mul1[want])
    torch.cuda.synchronize()
