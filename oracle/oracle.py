"""ctypes binding of the CPU oracle (oracle/t3_oracle.c). TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests, the smoke check and bench.py's cpu_baseline leg import this module; the package
``turboexl3_amd`` never does. numpy arrays in, numpy arrays out.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libt3oracle.so")

MUL1, MCG = 0, 1
CLAMP_GATE_IN, CLAMP_SILU_OUT = 0, 1


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libt3oracle.so"])
    return _LIB_PATH


class _Bank(C.Structure):
    _fields_ = [
        ("experts", C.c_size_t), ("hidden", C.c_size_t), ("inter", C.c_size_t),
        ("n_gu", C.c_uint32), ("n_dn", C.c_uint32),
        ("gate_t", C.c_void_p), ("gate_suh", C.c_void_p), ("gate_svh", C.c_void_p),
        ("up_t", C.c_void_p), ("up_suh", C.c_void_p), ("up_svh", C.c_void_p),
        ("down_t", C.c_void_p), ("down_suh", C.c_void_p), ("down_svh", C.c_void_p),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        u16p, u32p, f32p, i32p = (C.POINTER(C.c_uint16), C.POINTER(C.c_uint32), C.POINTER(C.c_float),
                                  C.POINTER(C.c_int32))
        sz, u32, i = C.c_size_t, C.c_uint32, C.c_int
        sig = {
            "t3o_f16_to_f32": (C.c_float, [C.c_uint16]),
            "t3o_f32_to_f16": (C.c_uint16, [C.c_float]),
            "t3o_f32_to_bf16": (C.c_uint16, [C.c_float]),
            "t3o_decode_mcg": (C.c_uint16, [C.c_uint16]),
            "t3o_decode_mul1": (C.c_uint16, [C.c_uint16]),
            "t3o_mul1_bytesum": (u32, [C.c_uint16]),
            "t3o_rate_ok": (i, [C.c_uint64]),
            "t3o_bit_end": (u32, [u32, u32]),
            "t3o_window_mask": (u32, [i]),
            "t3o_unpack_tile": (None, [u16p, u32, u16p]),
            "t3o_codeword_by_definition": (C.c_uint16, [u16p, u32, u32]),
            "t3o_lane_codewords": (None, [u16p, u32, u32, u16p]),
            "t3o_pack_symbols": (None, [u16p, u32, u16p]),
            "t3o_tensor_core_perm": (None, [u32p]),
            "t3o_decode_tile": (None, [u16p, u32, i, u32, u16p]),
            "t3o_reconstruct_inner": (None, [u16p, sz, sz, u32, i, u32, u16p]),
            "t3o_reconstruct_public": (i, [u16p, u16p, u16p, sz, sz, u32, i, u32, u16p]),
            "t3o_hadamard128": (None, [f32p]),
            "t3o_prepare_input": (None, [f32p, u16p, sz, f32p]),
            "t3o_inner_gemv": (None, [u16p, f32p, sz, sz, u32, i, u32, f32p]),
            "t3o_finish_output": (None, [f32p, u16p, sz, f32p]),
            "t3o_project": (None, [f32p, u16p, u16p, u16p, sz, sz, u32, i, u32, f32p]),
            "t3o_project_rows": (i, [f32p, sz, u16p, u16p, u16p, u16p, sz, sz, u32, i, u32, i, f32p]),
            "t3o_swiglu_clamped": (C.c_float, [C.c_float, C.c_float, C.c_float]),
            "t3o_swiglu_clamped_out": (C.c_float, [C.c_float, C.c_float, C.c_float]),
            "t3o_moe_row_clamped_at": (i, [C.POINTER(_Bank), i, u32, C.c_float, i, f32p, i32p, f32p, sz, f32p,
                                           C.POINTER(sz)]),
            "t3o_compare": (C.c_double, [f32p, f32p, sz, C.c_double]),
            "t3o_rb_cap": (u32, [u32, u32]),
            "t3o_bt_for": (u32, [u32]),
            "t3o_ks_for": (u32, [u32, u32]),
            "t3o_ks_gu": (u32, [u32, u32]),
            "t3o_ks_dn": (u32, [u32, u32]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a: np.ndarray, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16 or a.dtype == np.int16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


# ---- scalars and tables ---------------------------------------------------------------------------------

def decode_mcg(cw: int) -> int:
    return lib().t3o_decode_mcg(cw)


def decode_mul1(cw: int) -> int:
    return lib().t3o_decode_mul1(cw)


def mul1_bytesum(cw: int) -> int:
    return lib().t3o_mul1_bytesum(cw)


def codebook_table(codebook: int) -> np.ndarray:
    """All 65,536 codewords decoded: f16 bits as uint16."""
    fn = lib().t3o_decode_mcg if codebook == MCG else lib().t3o_decode_mul1
    return np.fromiter((fn(c) for c in range(65536)), dtype=np.uint16, count=65536)


def window_mask(bits: int) -> int:
    return lib().t3o_window_mask(bits)


def tensor_core_perm() -> np.ndarray:
    out = np.zeros(256, dtype=np.uint32)
    lib().t3o_tensor_core_perm(_p(out, C.c_uint32))
    return out


# ---- tiles ------------------------------------------------------------------------------------------------

def unpack_tile(words, n: int) -> np.ndarray:
    words = _u16(words)
    assert words.size == n
    out = np.zeros(256, dtype=np.uint16)
    lib().t3o_unpack_tile(_p(words, C.c_uint16), n, _p(out, C.c_uint16))
    return out


def codeword_by_definition(words, n: int, t: int) -> int:
    words = _u16(words)
    return lib().t3o_codeword_by_definition(_p(words, C.c_uint16), n, t)


def lane_codewords(words, n: int, lane: int) -> np.ndarray:
    words = _u16(words)
    out = np.zeros(8, dtype=np.uint16)
    lib().t3o_lane_codewords(_p(words, C.c_uint16), n, lane, _p(out, C.c_uint16))
    return out


def pack_symbols(symbols, k: int) -> np.ndarray:
    symbols = _u16(symbols)
    assert symbols.size == 256
    out = np.zeros(16 * k, dtype=np.uint16)
    lib().t3o_pack_symbols(_p(symbols, C.c_uint16), k, _p(out, C.c_uint16))
    return out


def decode_tile(words, n: int, codebook: int, mask: int = 0xFFFF) -> np.ndarray:
    words = _u16(words)
    out = np.zeros(256, dtype=np.uint16)
    lib().t3o_decode_tile(_p(words, C.c_uint16), n, codebook, mask, _p(out, C.c_uint16))
    return out


def reconstruct_inner(trellis, in_f: int, out_f: int, n: int, codebook: int, mask: int = 0xFFFF) -> np.ndarray:
    """W_hat [in, out] as f16 bits (uint16)."""
    trellis = _u16(trellis)
    assert trellis.size == (in_f // 16) * (out_f // 16) * n
    out = np.zeros((in_f, out_f), dtype=np.uint16)
    lib().t3o_reconstruct_inner(_p(trellis, C.c_uint16), in_f, out_f, n, codebook, mask, _p(out, C.c_uint16))
    return out


def reconstruct_public(trellis, suh, svh, in_f: int, out_f: int, n: int, codebook: int,
                       mask: int = 0xFFFF) -> np.ndarray:
    trellis, suh, svh = _u16(trellis), _u16(suh), _u16(svh)
    out = np.zeros((in_f, out_f), dtype=np.uint16)
    rc = lib().t3o_reconstruct_public(_p(trellis, C.c_uint16), _p(suh, C.c_uint16), _p(svh, C.c_uint16), in_f, out_f,
                                      n, codebook, mask, _p(out, C.c_uint16))
    assert rc == 0
    return out


# ---- projection ---------------------------------------------------------------------------------------

def hadamard128(v) -> np.ndarray:
    v = _f32(v).copy()
    assert v.size == 128
    lib().t3o_hadamard128(_p(v, C.c_float))
    return v


def prepare_input(x, suh) -> np.ndarray:
    x, suh = _f32(x), _u16(suh)
    out = np.zeros_like(x)
    lib().t3o_prepare_input(_p(x, C.c_float), _p(suh, C.c_uint16), x.size, _p(out, C.c_float))
    return out


def inner_gemv(trellis, transformed, in_f, out_f, n, codebook, mask=0xFFFF) -> np.ndarray:
    trellis, transformed = _u16(trellis), _f32(transformed)
    out = np.zeros(out_f, dtype=np.float32)
    lib().t3o_inner_gemv(_p(trellis, C.c_uint16), _p(transformed, C.c_float), in_f, out_f, n, codebook, mask,
                         _p(out, C.c_float))
    return out


def finish_output(inner, svh) -> np.ndarray:
    inner, svh = _f32(inner), _u16(svh)
    out = np.zeros_like(inner)
    lib().t3o_finish_output(_p(inner, C.c_float), _p(svh, C.c_uint16), inner.size, _p(out, C.c_float))
    return out


def project(x, trellis, suh, svh, in_f, out_f, n, codebook, mask=0xFFFF) -> np.ndarray:
    """One row through one projection, re-decoding every tile (format.project)."""
    x, trellis, suh, svh = _f32(x), _u16(trellis), _u16(suh), _u16(svh)
    assert x.size == in_f and suh.size == in_f and svh.size == out_f
    y = np.zeros(out_f, dtype=np.float32)
    lib().t3o_project(_p(x, C.c_float), _p(trellis, C.c_uint16), _p(suh, C.c_uint16), _p(svh, C.c_uint16), in_f,
                      out_f, n, codebook, mask, _p(y, C.c_float))
    return y


def project_rows(x, trellis, suh, svh, in_f, out_f, n, codebook, mask=0xFFFF, threads=1, w_hat=None) -> np.ndarray:
    """`rows` rows on a W_hat decoded once; the bits of `project` per row."""
    x, trellis, suh, svh = _f32(x).reshape(-1, in_f), _u16(trellis), _u16(suh), _u16(svh)
    rows = x.shape[0]
    y = np.zeros((rows, out_f), dtype=np.float32)
    wp = _p(_u16(w_hat), C.c_uint16) if w_hat is not None else None
    rc = lib().t3o_project_rows(_p(x, C.c_float), rows, _p(trellis, C.c_uint16), wp, _p(suh, C.c_uint16),
                                _p(svh, C.c_uint16), in_f, out_f, n, codebook, mask, threads, _p(y, C.c_float))
    assert rc == 0
    return y


# ---- routed experts -------------------------------------------------------------------------------------

@dataclass
class Bank:
    """ref.Bank: expert e on axis 0. Trellis uint16 [E, in/16, out/16, n]; suh/svh f16 bits [E, dim]."""
    experts: int
    hidden: int
    inter: int
    n_gu: int
    n_dn: int
    gate_t: np.ndarray
    gate_suh: np.ndarray
    gate_svh: np.ndarray
    up_t: np.ndarray
    up_suh: np.ndarray
    up_svh: np.ndarray
    down_t: np.ndarray
    down_suh: np.ndarray
    down_svh: np.ndarray

    def _c(self) -> _Bank:
        names = ["gate_t", "gate_suh", "gate_svh", "up_t", "up_suh", "up_svh", "down_t", "down_suh", "down_svh"]
        for nm in names:
            setattr(self, nm, _u16(getattr(self, nm)))
        b = _Bank(self.experts, self.hidden, self.inter, self.n_gu, self.n_dn)
        for nm in names:
            setattr(b, nm, getattr(self, nm).ctypes.data)
        return b


def moe_row(bank: Bank, x, slots, scores, codebook, mask=0xFFFF, limit=0.0, clamp_at=CLAMP_GATE_IN):
    """ref.moeRowClampedAt: y [hidden] and (gate hits, up hits, total)."""
    x = _f32(x)
    slots = np.ascontiguousarray(slots, dtype=np.int32)
    scores = _f32(scores)
    y = np.zeros(bank.hidden, dtype=np.float32)
    hits = (C.c_size_t * 3)()
    cb = bank._c()
    rc = lib().t3o_moe_row_clamped_at(C.byref(cb), codebook, mask, limit, clamp_at, _p(x, C.c_float),
                                      _p(slots, C.c_int32), _p(scores, C.c_float), slots.size, _p(y, C.c_float), hits)
    assert rc == 0
    return y, tuple(hits)


def compare(got, ref, half_ulp: float = 0.0) -> float:
    """ref.compare / compareRounded: max |got - ref| (beyond the store rounding) over rms(ref)."""
    got, ref = _f32(got).ravel(), _f32(ref).ravel()
    assert got.size == ref.size
    return lib().t3o_compare(_p(got, C.c_float), _p(ref, C.c_float), got.size, half_ulp)


# ---- synthetic data (ref.synthBank / synthLinear's distributions, numpy's generator) --------------------

def synth_linear(rng: np.random.Generator, in_f: int, out_f: int, n: int):
    """trellis uint16 [in/16, out/16, n] uniform; suh in [0.5, 1.5]; svh in [0.5, 1.5] / sqrt(in) (f16 bits)."""
    trellis = rng.integers(0, 65536, size=(in_f // 16, out_f // 16, n), dtype=np.uint16)
    suh = (0.5 + rng.random(in_f, dtype=np.float32)).astype(np.float16).view(np.uint16)
    svh = ((0.5 + rng.random(out_f, dtype=np.float32)) / np.sqrt(np.float32(in_f))).astype(np.float16).view(np.uint16)
    return trellis, suh, svh


def synth_bank(rng: np.random.Generator, experts: int, hidden: int, inter: int, n_gu: int, n_dn: int | None = None) -> Bank:
    n_dn = n_gu if n_dn is None else n_dn

    def stack(in_f, out_f, n):
        t = rng.integers(0, 65536, size=(experts, in_f // 16, out_f // 16, n), dtype=np.uint16)
        suh = (0.5 + rng.random((experts, in_f), dtype=np.float32)).astype(np.float16).view(np.uint16)
        svh = ((0.5 + rng.random((experts, out_f), dtype=np.float32)) / np.sqrt(np.float32(in_f))).astype(
            np.float16).view(np.uint16)
        return t, suh, svh

    g, u, d = stack(hidden, inter, n_gu), stack(hidden, inter, n_gu), stack(inter, hidden, n_dn)
    return Bank(experts, hidden, inter, n_gu, n_dn, g[0], g[1], g[2], u[0], u[1], u[2], d[0], d[1], d[2])
