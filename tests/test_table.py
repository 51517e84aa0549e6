"""The quant table's claim, validation, bill and load checks: the cases of the reference's own tests
(table/config.zig:160-204), plus the load checks' names (table/table.zig:128-174). Pure host logic: no GPU."""
import ctypes as C

import pytest

from turboexl3_amd import _lib

TRUNK = '{"format":"exl3","codebook":"mul1","window":16}'
BANK = '{"format":"exl3","k":5,"codebook":"mul1"}'
QWEN38 = '{"model_type":"qwen4_exp","trunk_quant":' + TRUNK + ',"text_config":{"num_experts_per_tok":8}}'
QWEN38_EXPERTS_ONLY = '{"model_type":"qwen4_exp","text_config":{"num_experts_per_tok":8}}'
GLM = '{"model_type":"glm5_next","swiglu_limit":7.0}'


@pytest.fixture(scope="module")
def L():
    return _lib.lib()


def claim(L, block, config, gate):
    return L.t3_table_claims(block.encode(), config.encode(), int(gate))


def verdict(L, block, config):
    buf = C.create_string_buffer(96)
    kind = L.t3_table_validate(block.encode(), config.encode(), buf, len(buf))
    return kind, buf.value.decode()


def test_claims(L):
    # table/config.zig:166-184
    for gate in (True, False):
        assert claim(L, TRUNK, "{}", gate) == _lib.CLAIM_BY_MARKER
    assert claim(L, BANK, QWEN38, True) == _lib.CLAIM_BY_MARKER
    assert claim(L, BANK, QWEN38, False) == _lib.CLAIM_NO
    assert claim(L, BANK, QWEN38_EXPERTS_ONLY, True) == _lib.CLAIM_NO
    assert claim(L, BANK, '{"model_type":"mimo_v2","trunk_quant":' + TRUNK + '}', True) == _lib.CLAIM_NO
    assert claim(L, BANK, GLM, True) == _lib.CLAIM_NO
    assert claim(L, '{"format":"stq","k":3,"codebook":"std1"}', QWEN38, True) == _lib.CLAIM_NO
    assert claim(L, '{"format":"exl3","k":3,"codebook":"pair1"}', QWEN38, True) == _lib.CLAIM_NO
    assert claim(L, '{"bits":4,"group_size":64}', QWEN38, True) == _lib.CLAIM_NO
    assert claim(L, "{}", "{}", True) == _lib.CLAIM_NO
    assert claim(L, "{", "{}", True) == _lib.CLAIM_NO
    # the text config may carry the model type; a clamp there counts too
    nested = '{"trunk_quant":' + TRUNK + ',"text_config":{"model_type":"qwen4_exp_text"}}'
    assert claim(L, BANK, nested, True) == _lib.CLAIM_BY_MARKER
    assert claim(L, BANK, nested.replace('"qwen4_exp_text"', '"qwen4_exp_text","swiglu_limit":7'), True) == _lib.CLAIM_NO
    assert claim(L, BANK, nested.replace('"qwen4_exp_text"', '"qwen4_exp_text","swiglu_limit":0'), True) == _lib.CLAIM_BY_MARKER


def test_validate_names(L):
    # table/config.zig:186-199
    assert verdict(L, TRUNK, "{}") == (_lib.VERDICT_OK, "")
    assert verdict(L, BANK, QWEN38) == (_lib.VERDICT_OK, "")
    assert verdict(L, '{"format":"exl3","codebook":"mcg","window":12}', "{}") == (_lib.VERDICT_OK, "")
    for block, config, want in (
        ('{"format":"exl3","codebook":"std1"}', "{}", "Exl3CodebookUnsupported"),
        ('{"format":"exl3","window":7}', "{}", "Exl3WindowUnsupported"),
        ('{"format":"exl3","k":1.03,"codebook":"mul1"}', "{}", "Exl3RateUnsupported"),
        ('{"format":"exl3","k":9,"codebook":"mul1"}', "{}", "Exl3RateUnsupported"),
        (BANK, '{"num_experts_per_tok":33}', "Exl3TopKExceedsReduceBank"),
        ('{"bits":4}', "{}", "NotExl3"),
        ('{"format":"exl3","k":3}', "{}", "Exl3CodebookUnsupported"),  # a bank block must name its codebook
        ('{"format":"exl3","window":"16"}', "{}", "Exl3WindowUnsupported"),
    ):
        assert verdict(L, block, config) == (_lib.VERDICT_UNSUPPORTED, want), block
    assert verdict(L, BANK, '{"text_config":{"num_experts_per_tok":32}}') == (_lib.VERDICT_OK, "")
    assert verdict(L, BANK, '{"text_config":{"num_experts_per_tok":40}}')[1] == "Exl3TopKExceedsReduceBank"
    # a reason longer than the buffer is truncated, never overrun
    buf = C.create_string_buffer(8)
    assert L.t3_table_validate(b'{"bits":4}', b"{}", buf, len(buf)) == _lib.VERDICT_UNSUPPORTED and buf.value == b"NotExl3"
    buf = C.create_string_buffer(4)
    L.t3_table_validate(b'{"bits":4}', b"{}", buf, len(buf))
    assert buf.value == b"Not"


def test_parse_block_rates(L):
    # table/config.zig:201-211
    b = _lib.Block()
    assert L.t3_table_parse_block(BANK.encode(), C.byref(b)) == 0
    assert (b.kind, b.n, b.codebook, b.window_bits) == (_lib.BLOCK_BANK, 80, 0, 16)
    assert L.t3_table_parse_block(b'{"format":"exl3","k":2.5,"codebook":"mcg","window":14}', C.byref(b)) == 0
    assert (b.n, b.codebook, b.window_bits) == (40, 1, 14)
    assert L.t3_table_parse_block(TRUNK.encode(), C.byref(b)) == 0
    assert (b.kind, b.n, b.window_bits) == (_lib.BLOCK_TRUNK, 0, 16)
    for k, n in (("1", 16), ("8", 128), ("2.25", 36), ("3.5", 56)):
        assert L.t3_table_parse_block(('{"format":"exl3","k":%s,"codebook":"mul1"}' % k).encode(), C.byref(b)) == 0 and b.n == n
    for k in ("0.5", "8.5", "2.0625", '"4"', "null"):  # under 16, over 128, an odd halfword count, not a number
        st = L.t3_table_parse_block(('{"format":"exl3","k":%s,"codebook":"mul1"}' % k).encode(), C.byref(b))
        assert L.t3_error_name(st) == b"Exl3RateUnsupported", k


def test_bill_is_the_stored_bytes(L):
    assert L.t3_table_bill(BANK.encode(), b"/models/x", 123456789012) == 123456789012


def arr(dtype, *shape, data=0x1000):
    a = _lib.Array()
    a.data, a.ndim, a.dtype = data, len(shape), dtype
    for i, d in enumerate(shape):
        a.shape[i] = d
    return a


def load(L, entry, block, a, b, c, in_dim=0):
    w = _lib.Weight()
    buf = C.create_string_buffer(96)
    ptr = lambda x: None if x is None else C.byref(x)
    kind = entry(C.byref(block), ptr(a), ptr(b), ptr(c), in_dim, C.byref(w), buf, len(buf))
    return kind, buf.value.decode(), w


def test_load_checks(L):
    trunk, bank = _lib.Block(), _lib.Block()
    L.t3_table_parse_block(b'{"format":"exl3","codebook":"mcg","window":12}', C.byref(trunk))
    L.t3_table_parse_block(BANK.encode(), C.byref(bank))
    t = arr(_lib.U16, 32, 16, 64)
    suh, svh = arr(_lib.F16, 512), arr(_lib.F16, 256)
    kind, why, w = load(L, L.t3_table_load_tensor, trunk, t, suh, svh)
    assert (kind, why) == (_lib.VERDICT_OK, "") and (w.layout, w.flags, w.block) == (1, 12, 64)
    assert load(L, L.t3_table_load_tensor, trunk, t, suh, svh, 512)[0] == _lib.VERDICT_OK
    cases = (
        ((bank, t, suh, svh, 0), _lib.VERDICT_UNSUPPORTED, "turboexl3: dense linears load under the trunk_quant block"),
        ((trunk, None, suh, svh, 0), _lib.VERDICT_FAILED, "MissingWeight"),
        ((trunk, arr(_lib.U16, 32, 16), suh, svh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),
        ((trunk, arr(_lib.F16, 32, 16, 64), suh, svh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),
        ((trunk, arr(_lib.U16, 32, 16, 63), suh, svh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3RateUnsupported"),
        ((trunk, arr(_lib.U16, 30, 16, 64), arr(_lib.F16, 480), svh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3WidthNotMultipleOf128"),
        ((trunk, t, suh, svh, 1024), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),
        ((trunk, t, arr(_lib.F16, 500), svh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3SideGeometry"),
        ((trunk, t, suh, arr(_lib.F32, 256), 0), _lib.VERDICT_UNSUPPORTED, "Exl3SideDtype"),
    )
    for args, kind, why in cases:
        got = load(L, L.t3_table_load_tensor, *args)
        assert got[:2] == (kind, why), why
    # banks: trellis U16 [E, in/16, out/16, n] at or under the block's rate (80)
    bt = arr(_lib.U16, 8, 32, 16, 80)
    bsuh, bsvh = arr(_lib.F16, 8, 512), arr(_lib.F16, 8, 256)
    kind, why, w = load(L, L.t3_table_load_bank, bank, bt, bsuh, bsvh)
    assert (kind, why) == (_lib.VERDICT_OK, "") and (w.layout, w.flags, w.block) == (0, 16, 80)
    assert load(L, L.t3_table_load_bank, bank, arr(_lib.U16, 8, 32, 16, 64), bsuh, bsvh)[0] == _lib.VERDICT_OK
    for args, kind, why in (
        ((trunk, bt, bsuh, bsvh, 0), _lib.VERDICT_UNSUPPORTED, "turboexl3: routed banks load under the expert_quant block"),
        ((bank, bt, None, bsvh, 0), _lib.VERDICT_FAILED, "MissingWeight"),
        ((bank, arr(_lib.U16, 8, 32, 16, 96), bsuh, bsvh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),  # over the rate
        ((bank, arr(_lib.I16, 8, 32, 16, 80), bsuh, bsvh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),
        ((bank, bt, bsuh, bsvh, 256), _lib.VERDICT_UNSUPPORTED, "Exl3TrellisGeometry"),
        ((bank, bt, arr(_lib.F16, 8, 500), bsvh, 0), _lib.VERDICT_UNSUPPORTED, "Exl3SideGeometry"),
        ((bank, bt, bsuh, arr(_lib.F32, 8, 256), 0), _lib.VERDICT_UNSUPPORTED, "Exl3SideDtype"),
    ):
        assert load(L, L.t3_table_load_bank, *args)[:2] == (kind, why), why


def test_moe_refuses_and_swiglu_refuses_mixed_decodes(L):
    buf = C.create_string_buffer(96)
    assert L.t3_table_moe(buf, len(buf)) == _lib.VERDICT_UNSUPPORTED
    assert buf.value == b"turboexl3: a layer's banks run as one routed SwiGLU (swiglu)"
    bank, other = _lib.Block(), _lib.Block()
    L.t3_table_parse_block(BANK.encode(), C.byref(bank))
    L.t3_table_parse_block(b'{"format":"exl3","k":5,"codebook":"mcg"}', C.byref(other))
    gu = lambda blk: load(L, L.t3_table_load_bank, blk, arr(_lib.U16, 8, 32, 16, 80), arr(_lib.F16, 8, 512), arr(_lib.F16, 8, 256))[2]
    dn = lambda blk: load(L, L.t3_table_load_bank, blk, arr(_lib.U16, 8, 16, 32, 80), arr(_lib.F16, 8, 256), arr(_lib.F16, 8, 512))[2]
    x, inds, scores, y = arr(_lib.F16, 1, 1, 512), arr(_lib.I32, 1, 1, 2), arr(_lib.F32, 1, 1, 2), arr(_lib.F16, 1, 1, 512)
    g, u, d = gu(bank), gu(bank), dn(other)
    kind = L.t3_table_swiglu(None, C.byref(g), C.byref(u), C.byref(d), C.byref(x), C.byref(inds), C.byref(scores), 0, 0,
                             C.byref(y), None, 0, buf, len(buf))
    assert (kind, buf.value) == (_lib.VERDICT_UNSUPPORTED, b"turboexl3: a layer's banks decode differently")
    blank = _lib.Weight()
    kind = L.t3_table_swiglu(None, C.byref(blank), C.byref(u), C.byref(d), C.byref(x), C.byref(inds), C.byref(scores), 0, 0,
                             C.byref(y), None, 0, buf, len(buf))
    assert (kind, buf.value) == (_lib.VERDICT_FAILED, b"turboexl3: a bank without its decode")
    # a clamp past 128 is refused by name before anything launches (no workspace is passed here: nothing ran)
    g, u, d = gu(bank), gu(bank), dn(bank)
    kind = L.t3_table_swiglu(None, C.byref(g), C.byref(u), C.byref(d), C.byref(x), C.byref(inds), C.byref(scores), 129, 0,
                             C.byref(y), None, 0, buf, len(buf))
    assert (kind, buf.value) == (_lib.VERDICT_UNSUPPORTED, b"InvalidExl3Clamp")
