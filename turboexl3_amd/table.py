"""turboexl3 as a quant table (the reference's table/config.zig and table/table.zig) over the C ABI's `t3_table_*`
entry points: claims, validation, the bill, weight loading checks, and `matmul` / `swiglu` over loaded weights."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .api import _arr, _stream_ptr, _workspace

NAME = "turboexl3"  # table/table.zig:27


class Refused(Exception):
    """A verdict other than ok: `kind` ('unsupported' / 'failed' / 'too_large') and the reference's reason."""

    def __init__(self, kind: int, why: str):
        self.kind = {1: "unsupported", 2: "failed", 3: "too_large"}.get(kind, str(kind))
        self.why = why
        super().__init__(f"{self.kind}: {why}")


def _verdict(kind: int, buf) -> None:
    if kind != _lib.VERDICT_OK:
        raise Refused(kind, buf.value.decode())


def parse_block(block_json: str) -> _lib.Block:
    b = _lib.Block()
    st = _lib.lib().t3_table_parse_block(block_json.encode(), C.byref(b))
    if st != 0:
        raise ValueError(_lib.error_name(st))
    return b


def claims(block_json: str, config_json: str, matrix_gate: bool = True) -> str:
    return ("no", "by_type", "by_marker")[_lib.lib().t3_table_claims(block_json.encode(), config_json.encode(), int(matrix_gate))]


def validate(block_json: str, config_json: str) -> None:
    buf = C.create_string_buffer(128)
    _verdict(_lib.lib().t3_table_validate(block_json.encode(), config_json.encode(), buf, len(buf)), buf)


def bill(block_json: str, model_dir: str, stored: int) -> int:
    return _lib.lib().t3_table_bill(block_json.encode(), model_dir.encode(), stored)


def _opt(t):
    return (None, None) if t is None else (lambda a: (C.byref(a), a))(_arr(t))


def _load(entry, block: _lib.Block, a, b, c, in_dim: int) -> _lib.Weight:
    w = _lib.Weight()
    buf = C.create_string_buffer(128)
    (pa, ka), (pb, kb), (pc, kc) = _opt(a), _opt(b), _opt(c)
    _verdict(entry(C.byref(block), pa, pb, pc, in_dim, C.byref(w), buf, len(buf)), buf)
    w._keep = (ka, kb, kc)
    return w


def load_tensor(block: _lib.Block, weight, scales, biases, in_dim: int = 0) -> _lib.Weight:
    return _load(_lib.lib().t3_table_load_tensor, block, weight, scales, biases, in_dim)


def load_bank(block: _lib.Block, trellis, suh, svh, in_dim: int = 0) -> _lib.Weight:
    return _load(_lib.lib().t3_table_load_bank, block, trellis, suh, svh, in_dim)


def matmul(w: _lib.Weight, x: torch.Tensor, stream=None) -> torch.Tensor:
    L = _lib.lib()
    ax = _arr(x)
    need = C.c_size_t(0)
    st = L.t3_table_matmul_workspace_bytes(C.byref(w), C.byref(ax), C.byref(need))
    if st != 0:
        raise Refused(_lib.VERDICT_UNSUPPORTED, _lib.error_name(st))
    y = torch.empty(*x.shape[:-1], w.w.shape[1] * 16, dtype=x.dtype, device=x.device)
    ay = _arr(y)
    ws = _workspace(x.device, need.value)
    buf = C.create_string_buffer(128)
    _verdict(L.t3_table_matmul(_stream_ptr(stream), C.byref(w), C.byref(ax), C.byref(ay), ws.data_ptr(), ws.numel(), buf,
                               len(buf)), buf)
    return y


def moe() -> None:
    buf = C.create_string_buffer(128)
    _verdict(_lib.lib().t3_table_moe(buf, len(buf)), buf)


def swiglu(gate: _lib.Weight, up: _lib.Weight, down: _lib.Weight, x, inds, scores, limit: int = 0,
           verify_rows: bool = False, stream=None) -> torch.Tensor:
    L = _lib.lib()
    ax, ai, asc = _arr(x), _arr(inds), _arr(scores)
    need = C.c_size_t(0)
    buf = C.create_string_buffer(128)
    y = torch.empty_like(x)
    ay = _arr(y)
    st = L.t3_table_swiglu_workspace_bytes(C.byref(gate), C.byref(up), C.byref(down), C.byref(ax), C.byref(ai), C.byref(need))
    ws = _workspace(x.device, need.value if st == 0 else 0)
    _verdict(L.t3_table_swiglu(_stream_ptr(stream), C.byref(gate), C.byref(up), C.byref(down), C.byref(ax), C.byref(ai),
                               C.byref(asc), limit, int(verify_rows), C.byref(ay), ws.data_ptr(), ws.numel(), buf, len(buf)),
             buf)
    return y
