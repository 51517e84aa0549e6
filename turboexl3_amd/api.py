"""The module entry points of turboexl3's projection path over torch device tensors, mirroring
src/root.zig's `linear` (:309-351), `moe` (:822-904), `moeWithShared` (:976-984), `moeClamped` (:1001-1004) and
`configure`: same names, argument meaning and refusals (a refusal raises `T3Error` carrying the reference's
error name). torch is plumbing here: it owns device memory and the stream; all arithmetic runs in
libturboexl3_hip.so through the C ABI."""
from __future__ import annotations

import ctypes as C
import threading
from dataclasses import dataclass

import torch

from . import _lib
from ._lib import Array, Bank as CBank, Config, Decode as CDecode, Proj as CProj

MUL1, MCG = 0, 1


class T3Error(RuntimeError):
    """A named refusal or failure; `.name` is the reference's Zig error name."""

    def __init__(self, status: int):
        self.status = status
        self.name = _lib.error_name(status)
        super().__init__(self.name)


@dataclass(frozen=True)
class Decode:
    """format.Decode: codebook (0 MUL1 / 1 MCG) and codeword window (8..16 bits)."""
    codebook: int = MUL1
    window_bits: int = 16

    def c(self) -> CDecode:
        return CDecode(self.codebook, self.window_bits)


Decode.mul1 = Decode(MUL1, 16)
Decode.mcg = Decode(MCG, 16)


@dataclass
class Proj:
    """One projection's arrays (root.Proj): trellis U16/I16 [E, in/16, out/16, n], suh F16 [E, in], svh F16 [E, out]."""
    trellis: torch.Tensor
    suh: torch.Tensor
    svh: torch.Tensor


@dataclass
class Bank:
    gate: Proj
    up: Proj
    down: Proj


_DTYPES = {
    torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16,
    torch.uint16: _lib.U16, torch.int16: _lib.I16, torch.uint32: _lib.U32, torch.int32: _lib.I32,
}


def _arr(t: torch.Tensor) -> Array:
    if not isinstance(t, torch.Tensor):
        raise TypeError("expected a torch.Tensor")
    if t.dtype not in _DTYPES:
        raise T3Error(2)  # BadExl3Dtype
    if t.dim() > _lib.T3_MAX_DIMS:
        raise T3Error(1)
    if not t.is_cuda:
        raise ValueError("turboexl3_amd runs on device tensors only")
    if not t.is_contiguous():
        t = t.contiguous()
    a = Array()
    a.data = t.data_ptr()
    a.ndim = t.dim()
    a.dtype = _DTYPES[t.dtype]
    for i, d in enumerate(t.shape):
        a.shape[i] = d
    a._keep = t
    return a


def _check(status: int) -> None:
    if status != 0:
        raise T3Error(status)


def _stream_ptr(stream) -> int:
    s = torch.cuda.current_stream() if stream is None else stream
    return s.cuda_stream


_workspaces: dict = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """A grow-only scratch buffer per device and host thread (the caller of the C ABI owns scratch; calls that share a
    workspace must be ordered on one stream, so every thread of this harness keeps its own)."""
    key = (device.type, device.index, threading.get_ident())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        # zero-filled once: the head of a workspace holds the fused launches' arrival counters
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def configure(**fields) -> None:
    """root.configure: set once before the first call; an unserved value raises InvalidTurboexl3Config."""
    cfg = Config()
    _lib.lib().t3_config_default(C.byref(cfg))
    for k, v in fields.items():
        if not hasattr(cfg, k):
            raise T3Error(10)
        setattr(cfg, k, int(v))
    _check(_lib.lib().t3_configure(C.byref(cfg)))


def release_engines() -> None:
    _lib.lib().t3_release_engines()


def _linear(entry, x, trellis, suh, svh, dec: Decode, stream=None) -> torch.Tensor:
    L = _lib.lib()
    ax, at, asu, asv = _arr(x), _arr(trellis), _arr(suh), _arr(svh)
    need = C.c_size_t(0)
    _check(L.t3_linear_workspace_bytes(C.byref(ax), C.byref(at), dec.c(), C.byref(need)))
    out_dim = trellis.shape[1] * 16
    y = torch.empty(*x.shape[:-1], out_dim, dtype=x.dtype, device=x.device)
    ay = _arr(y)
    ws = _workspace(x.device, need.value)
    _check(entry(_stream_ptr(stream), C.byref(ax), C.byref(at), C.byref(asu), C.byref(asv), dec.c(), C.byref(ay),
                 ws.data_ptr(), ws.numel()))
    return y


def _plan_dict(p) -> dict:
    return {name: getattr(p, name) for name, _ in p._fields_}


def linear_plan(x, trellis, dec: Decode = Decode.mul1) -> dict:
    """How `linear` would run this call (path, launches, K slices, tiles a wave, workgroups, bytes): nothing is launched."""
    p = _lib.LinearPlan()
    ax, at = _arr(x), _arr(trellis)
    _check(_lib.lib().t3_linear_plan_of(C.byref(ax), C.byref(at), dec.c(), C.byref(p)))
    return _plan_dict(p)


def moe_plan(x, bank: "Bank", inds, shared_bank=None) -> dict:
    """How the routed entry points would run this call: nothing is launched."""
    p = _lib.MoePlan()
    ax, ai = _arr(x), _arr(inds)
    cb, _keep = _cbank(bank)
    sb = _cbank(shared_bank) if shared_bank is not None else None
    _check(_lib.lib().t3_moe_plan_of(C.byref(ax), C.byref(cb), C.byref(ai), C.byref(sb[0]) if sb else None, C.byref(p)))
    return _plan_dict(p)


def linear(x, trellis, suh, svh, dec: Decode = Decode.mul1, stream=None) -> torch.Tensor:
    """root.linear: y [..., out] in x's dtype for x [..., in]."""
    return _linear(_lib.lib().t3_linear, x, trellis, suh, svh, dec, stream)


def linear_static(x, trellis, suh, svh, dec: Decode = Decode.mul1, stream=None, out=None) -> torch.Tensor:
    """`linear` at decode rows through the entry point that allocates nothing: its scratch is the library's own device
    array (16 MiB a GPU). `out`: the caller's y (this harness allocates one otherwise; the C call never does)."""
    ax, at, asu, asv = _arr(x), _arr(trellis), _arr(suh), _arr(svh)
    y = out if out is not None else torch.empty(*x.shape[:-1], trellis.shape[1] * 16, dtype=x.dtype, device=x.device)
    ay = _arr(y)
    _check(_lib.lib().t3_linear_static(_stream_ptr(stream), C.byref(ax), C.byref(at), C.byref(asu), C.byref(asv), dec.c(),
                                       C.byref(ay)))
    return y


def linear_static_reset(stream=None) -> None:
    """Zero the counter head of the library's own scratch array again (after a call that did not run to its end)."""
    _check(_lib.lib().t3_linear_static_reset(_stream_ptr(stream)))


def linear_chain(x, trellis, suh, svh, dec: Decode = Decode.mul1, stream=None) -> torch.Tensor:
    """The three-launch chain `linear`'s fused launch must equal byte for byte."""
    return _linear(_lib.lib().t3_linear_chain, x, trellis, suh, svh, dec, stream)


def dequant(trellis, dec: Decode = Decode.mul1, stream=None) -> torch.Tensor:
    """W_hat f16 [in, out]: format.reconstructInner on the device, bit-exact."""
    at = _arr(trellis)
    if trellis.dim() != 3:
        raise T3Error(1)
    w = torch.empty(trellis.shape[0] * 16, trellis.shape[1] * 16, dtype=torch.float16, device=trellis.device)
    aw = _arr(w)
    _check(_lib.lib().t3_dequant(_stream_ptr(stream), C.byref(at), dec.c(), C.byref(aw)))
    return w


def linear_resident(x, w_hat, suh, svh, stream=None) -> torch.Tensor:
    """`linear` above 32 rows over a kept W_hat (`dequant`'s output): prepare, one plain f16 GEMM, finish."""
    L = _lib.lib()
    ax, aw, asu, asv = _arr(x), _arr(w_hat), _arr(suh), _arr(svh)
    need = C.c_size_t(0)
    _check(L.t3_linear_resident_workspace_bytes(C.byref(ax), C.byref(aw), C.byref(need)))
    y = torch.empty(*x.shape[:-1], w_hat.shape[1], dtype=x.dtype, device=x.device)
    ay = _arr(y)
    ws = _workspace(x.device, need.value)
    _check(L.t3_linear_resident(_stream_ptr(stream), C.byref(ax), C.byref(aw), C.byref(asu), C.byref(asv), C.byref(ay),
                                ws.data_ptr(), ws.numel()))
    return y


def unrot_weight(trellis, suh, svh, dec: Decode = Decode.mul1, dtype=torch.bfloat16, into=None, col0: int = 0,
                 stream=None):
    """The un-rotated weight W_std [in, out] in `dtype` (dense.unrotWeight), or written into columns col0.. of `into`
    (a join: one [in, N] array, its members side by side). Returns (w_std, nonfinite count)."""
    L = _lib.lib()
    at = _arr(trellis)
    if trellis.dim() != 3:
        raise T3Error(1)
    in_f, out_f = trellis.shape[0] * 16, trellis.shape[1] * 16
    w = into if into is not None else torch.empty(in_f, out_f, dtype=dtype, device=trellis.device)
    need = C.c_size_t(0)
    _check(L.t3_unrot_workspace_bytes(C.byref(at), C.byref(need)))
    ws = _workspace(trellis.device, need.value)
    bad = torch.zeros(1, dtype=torch.int32, device=trellis.device)
    asu, asv, aw = _arr(suh), _arr(svh), _arr(w)
    _check(L.t3_unrot_weight(_stream_ptr(stream), C.byref(at), C.byref(asu), C.byref(asv), dec.c(), C.byref(aw), col0,
                             bad.data_ptr(), ws.data_ptr(), ws.numel()))
    return w, int(bad.item())


def linear_unrot(x, w_std, col0: int = 0, cols=None, stream=None) -> torch.Tensor:
    """y = x W_std[:, col0 : col0 + cols]: one plain GEMM in the activation dtype (above 32 rows)."""
    cols = w_std.shape[1] - col0 if cols is None else cols
    y = torch.empty(*x.shape[:-1], cols, dtype=x.dtype, device=x.device)
    ax, aw, ay = _arr(x), _arr(w_std), _arr(y)
    _check(_lib.lib().t3_linear_unrot(_stream_ptr(stream), C.byref(ax), C.byref(aw), col0, cols, C.byref(ay)))
    return y


def linear_unrot_parts(x, w_std, col0: int = 0, cols=None, stream=None) -> torch.Tensor:
    """`linear_unrot` with K shared out over the grid where the GEMM's tiles are few (calls of few rows)."""
    L = _lib.lib()
    cols = w_std.shape[1] - col0 if cols is None else cols
    y = torch.empty(*x.shape[:-1], cols, dtype=x.dtype, device=x.device)
    ax, aw, ay = _arr(x), _arr(w_std), _arr(y)
    need = C.c_size_t(0)
    _check(L.t3_linear_unrot_workspace_bytes(C.byref(ax), C.byref(aw), col0, cols, C.byref(need)))
    ws = _workspace(x.device, need.value)
    _check(L.t3_linear_unrot_parts(_stream_ptr(stream), C.byref(ax), C.byref(aw), col0, cols, C.byref(ay), ws.data_ptr(),
                                   ws.numel()))
    return y


def _cbank(bank: Bank):
    keep = []

    def proj(p: Proj) -> CProj:
        a = (_arr(p.trellis), _arr(p.suh), _arr(p.svh))
        keep.append(a)
        return CProj(*a)

    return CBank(proj(bank.gate), proj(bank.up), proj(bank.down)), keep


def _moe_workspace(L, ax, cb, ai, device, shared=None):
    need = C.c_size_t(0)
    _check(L.t3_moe_workspace_bytes(C.byref(ax), C.byref(cb), C.byref(ai), C.byref(shared) if shared is not None else None,
                                    C.byref(need)))
    return _workspace(device, need.value)


def moe(x, bank: Bank, inds, scores, dec: Decode = Decode.mul1, verify_rows: bool = False, stream=None) -> torch.Tensor:
    """root.moe: routed SwiGLU experts over x [B, S, D] for inds/scores [B, S, K]."""
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    cb, _keep = _cbank(bank)
    ws = _moe_workspace(L, ax, cb, ai, x.device)
    y = torch.empty_like(x)
    ay = _arr(y)
    _check(L.t3_moe(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(),
                    int(verify_rows), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def moe_clamped(x, bank: Bank, inds, scores, dec: Decode, limit: int, stream=None) -> torch.Tensor:
    """root.moeClamped: gate clamped from above, up to [-limit, limit]; limit 1..128."""
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    cb, _keep = _cbank(bank)
    if not (0 < int(limit) <= 128):
        raise T3Error(6)
    ws = _moe_workspace(L, ax, cb, ai, x.device)
    y = torch.empty_like(x)
    ay = _arr(y)
    _check(L.t3_moe_clamped(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(),
                            int(limit), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


GATE_IN, SILU_OUT = 0, 1


def moe_swiglu(x, bank: Bank, inds, scores, dec: Decode, limit: int, clamp_at: int = GATE_IN, stream=None) -> torch.Tensor:
    """root.moeSwiglu: `moe` with the SwiGLU's clamp `limit` (0: none) at `clamp_at` (format.ClampAt)."""
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    cb, _keep = _cbank(bank)
    if not (0 <= int(limit) <= 128) or clamp_at not in (GATE_IN, SILU_OUT):
        raise T3Error(6)
    ws = _moe_workspace(L, ax, cb, ai, x.device)
    y = torch.empty_like(x)
    ay = _arr(y)
    _check(L.t3_moe_swiglu(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(), int(limit),
                           int(clamp_at), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def linear_bias(x, trellis, suh, svh, bias, dec: Decode = Decode.mul1, stream=None) -> torch.Tensor:
    """root.linearBias: `linear` plus a bias [out] in x's dtype (one add after the output rounding)."""
    L = _lib.lib()
    ax, at, asu, asv, ab = _arr(x), _arr(trellis), _arr(suh), _arr(svh), _arr(bias)
    need = C.c_size_t(0)
    _check(L.t3_linear_workspace_bytes(C.byref(ax), C.byref(at), dec.c(), C.byref(need)))
    y = torch.empty(*x.shape[:-1], trellis.shape[1] * 16, dtype=x.dtype, device=x.device)
    ay = _arr(y)
    ws = _workspace(x.device, need.value)
    _check(L.t3_linear_bias(_stream_ptr(stream), C.byref(ax), C.byref(at), C.byref(asu), C.byref(asv), C.byref(ab), dec.c(),
                            C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def moe_with_shared(x, bank: Bank, inds, scores, dec: Decode, verify_rows: bool, shared, stream=None) -> torch.Tensor:
    """root.moeWithShared: `moe` plus an already gated shared-expert output of x's shape and dtype."""
    L = _lib.lib()
    ax, ai, asc, ash = _arr(x), _arr(inds), _arr(scores), _arr(shared)
    cb, _keep = _cbank(bank)
    ws = _moe_workspace(L, ax, cb, ai, x.device)
    y = torch.empty_like(x)
    ay = _arr(y)
    _check(L.t3_moe_with_shared(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(),
                                int(verify_rows), C.byref(ash), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def moe_shared_expert(x, bank: Bank, inds, scores, dec: Decode, limit: int, shared_bank: Bank, stream=None) -> torch.Tensor:
    """The routed experts with every expert of `shared_bank` as extra slots of each row at weight 1 (limit 0: no clamp)."""
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    cb, _keep = _cbank(bank)
    sb, _keep2 = _cbank(shared_bank)
    ws = _moe_workspace(L, ax, cb, ai, x.device, sb)
    y = torch.empty_like(x)
    ay = _arr(y)
    _check(L.t3_moe_shared_expert(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(),
                                  int(limit), C.byref(sb), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def moe_fused_shared(x, bank: Bank, inds, scores, dec: Decode, shared_bank: Bank, sigtab, logit, stream=None) -> torch.Tensor:
    """qwen38's moeFusedShared at decode rows: routed + sigmoid(logit) * shared(x) inside the routed launches; sigtab
    [65536] in x's dtype (the sigmoid of every 16-bit pattern), logit [rows] in x's dtype."""
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    cb, _keep = _cbank(bank)
    sb, _keep2 = _cbank(shared_bank)
    ws = _moe_workspace(L, ax, cb, ai, x.device, sb)
    y = torch.empty_like(x)
    ay, at, al = _arr(y), _arr(sigtab), _arr(logit)
    _check(L.t3_moe_fused_shared(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), C.byref(asc), dec.c(),
                                 C.byref(sb), C.byref(at), C.byref(al), C.byref(ay), ws.data_ptr(), ws.numel()))
    return y


def moe_fused_shared_routed(x, bank: Bank, logits, k: int, dec: Decode, shared_bank: Bank, sigtab, logit, stream=None,
                            return_routing: bool = False, gate_vec=None):
    """qwen38's moeFusedSharedRouted: `moe_fused_shared` with the top-k and the renormalised softmax weights computed
    from the router's logits [B, S, E] by one launch in front. `logit` [rows], or None with `gate_vec` bf16 [D]: the
    shared gate's logit is then taken in the same launch. return_routing: also the slots and weights it made (and, with
    gate_vec, the logits)."""
    L = _lib.lib()
    ax, al = _arr(x), _arr(logits)
    cb, _keep = _cbank(bank)
    sb, _keep2 = _cbank(shared_bank)
    need = C.c_size_t(0)
    _check(L.t3_moe_fused_shared_routed_workspace_bytes(C.byref(ax), C.byref(cb), C.byref(al), int(k), C.byref(sb),
                                                        C.byref(need)))
    ws = _workspace(x.device, need.value)
    y = torch.empty_like(x)
    ay, at = _arr(y), _arr(sigtab)
    ag = _arr(logit) if logit is not None else None
    av = _arr(gate_vec) if gate_vec is not None else None
    _check(L.t3_moe_fused_shared_routed(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(al), int(k), dec.c(),
                                        C.byref(sb), C.byref(at), C.byref(ag) if ag is not None else None,
                                        C.byref(av) if av is not None else None, C.byref(ay), ws.data_ptr(), ws.numel()))
    if not return_routing:
        return y
    rows = x.shape[0] * x.shape[1]
    slots = rows * k
    pad = lambda b: (b + 255) & ~255
    tail = need.value - pad(slots * 4) - pad(slots * 2) - 256
    inds = ws[tail:tail + slots * 4].view(torch.int32).reshape(rows, k).clone()
    scores = ws[tail + pad(slots * 4):tail + pad(slots * 4) + slots * 2].view(x.dtype).reshape(rows, k).clone()
    if gate_vec is None:
        return y, inds, scores
    glogit = ws[need.value - 256:need.value - 256 + rows * 2].view(torch.bfloat16).clone()
    return y, inds, scores, glogit


def moe_glm(x, bank: Bank, inds, dec: Decode, limit: int = 0, stream=None, fill: float = 0.0) -> torch.Tensor:
    """The routed experts under GLM's rounding profile: x bf16 [B, S, D] -> f32 [B, S, K, D], a slot's own output each
    (a skipped slot keeps `fill`)."""
    L = _lib.lib()
    ax, ai = _arr(x), _arr(inds)
    cb, _keep = _cbank(bank)
    ws = _moe_workspace(L, ax, cb, ai, x.device)
    y = torch.full((x.shape[0], x.shape[1], inds.shape[2], x.shape[2]), fill, dtype=torch.float32, device=x.device)
    ay = _arr(y)
    _check(L.t3_moe_glm(_stream_ptr(stream), C.byref(ax), C.byref(cb), C.byref(ai), dec.c(), int(limit), C.byref(ay),
                        ws.data_ptr(), ws.numel()))
    return y


# ---- device self-tests -------------------------------------------------------------------------------------

def test_codebooks(device="cuda"):
    mcg = torch.empty(65536, dtype=torch.int16, device=device)
    mul1 = torch.empty_like(mcg)
    t = torch.empty_like(mcg)
    _check(_lib.lib().t3_test_codebooks(_stream_ptr(None), mcg.data_ptr(), mul1.data_ptr(), t.data_ptr()))
    return mcg, mul1, t


def test_lane(trellis: torch.Tensor, n: int, window_bits: int):
    tiles = trellis.numel() // n
    cw = torch.empty(tiles, 256, dtype=torch.int16, device=trellis.device)
    mcg = torch.empty_like(cw)
    mul1 = torch.empty_like(cw)
    _check(_lib.lib().t3_test_lane(_stream_ptr(None), trellis.data_ptr(), n, window_bits, tiles, cw.data_ptr(),
                                   mcg.data_ptr(), mul1.data_ptr()))
    return cw, mcg, mul1


def test_convert(values: torch.Tensor):
    """f32 values through the kernels' narrowing: (bf16 bits, f16 bits, the bf16 widened back to f32)."""
    n = values.numel()
    bf = torch.empty(n, dtype=torch.int16, device=values.device)
    hf = torch.empty_like(bf)
    back = torch.empty(n, dtype=torch.float32, device=values.device)
    _check(_lib.lib().t3_test_convert(_stream_ptr(None), values.data_ptr(), bf.data_ptr(), hf.data_ptr(), back.data_ptr(), n))
    return bf, hf, back


def test_mfma(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    d = torch.empty(16, 16, dtype=torch.float32, device=a.device)
    _check(_lib.lib().t3_test_mfma(_stream_ptr(None), a.data_ptr(), b.data_ptr(), d.data_ptr()))
    return d
