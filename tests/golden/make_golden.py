#!/usr/bin/env python3
"""Writes tests/golden/exl3_golden.json: small known-answer vectors of the EXL3 format.

Nothing here imports the oracle, the library or the reference: every vector comes from the format's definition
restated with numpy (bit-by-bit stream reads, numpy float16 arithmetic), or is a literal the reference's own tests
hold (cited). The tests hold the C oracle and the device kernels to this file.

    python tests/golden/make_golden.py
"""
import hashlib
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
RATES = [16, 32, 36, 40, 48, 64, 80, 96, 128]


def mcg_table() -> np.ndarray:
    """format.decodeMcg (turboexl3 src/core/format.zig:149-155) for every codeword."""
    cw = np.arange(65536, dtype=np.uint64)
    mixed = (cw * 0xCBAC1FED) & 0xFFFFFFFF
    pair = (0x3B603B60 ^ (mixed & 0x8FFF8FFF)).astype(np.uint32)
    lo = (pair & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
    hi = (pair >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
    return (lo + hi).astype(np.float16).view(np.uint16)


def mul1_table() -> np.ndarray:
    """format.decodeMul1 (src/core/format.zig:158-167): the exact value fits 20 bits, so f64 then one rounding."""
    cw = np.arange(65536, dtype=np.uint64)
    mixed = ((cw * 0x83DCD12D) & 0xFFFFFFFF).astype(np.uint32)
    t = mixed.view(np.uint8).reshape(-1, 4).astype(np.uint32).sum(axis=1)
    h = (0x6400 + t).astype(np.uint16).view(np.float16).astype(np.float64)
    a = np.array([0x1EEE], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    b = np.array([0xC931], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    return (h * a + b).astype(np.float16).view(np.uint16)


def codewords_by_definition(tile: np.ndarray) -> np.ndarray:
    """The 256 codewords of one packed tile, read bit by bit (src/core/format.zig:204-222): u16 pairs are
    little-endian u32 words, stream bit j is bit 31 - j % 32 of word j / 32, the stream is circular, and codeword t
    is the 16 bits ending at bit ((t + 1) n) >> 4."""
    n = tile.size
    words = tile.astype(np.uint32).reshape(-1, 2)
    words = words[:, 0] | (words[:, 1] << 16)
    bits = np.array([(int(words[j // 32]) >> (31 - j % 32)) & 1 for j in range(16 * n)], dtype=np.uint32)
    out = np.zeros(256, dtype=np.uint16)
    for t in range(256):
        end = ((t + 1) * n) >> 4
        v = 0
        for k in range(16):
            v = (v << 1) | int(bits[(end - 16 + k) % (16 * n)])
        out[t] = v
    return out


def tensor_core_perm() -> list:
    """Code position p = 8 L + i -> row-major tile index (src/core/format.zig:237-256): rows 2 (L % 4) + {0, 1, 8, 9}
    [i % 4], column L / 4 + 8 (i / 4)."""
    perm = []
    for p in range(256):
        lane, i = p // 8, p % 8
        row = 2 * (lane % 4) + (0, 1, 8, 9)[i % 4]
        col = lane // 4 + 8 * (i // 4)
        perm.append(row * 16 + col)
    return perm


def main() -> None:
    rng = np.random.default_rng(0x601D)
    tiles = {}
    for n in RATES:
        tile = rng.integers(0, 65536, n, dtype=np.uint16)
        tiles[str(n)] = {"trellis_u16": tile.tolist(), "codewords": codewords_by_definition(tile).tolist()}
    mcg, mul1 = mcg_table(), mul1_table()
    golden = {
        "about": "EXL3 format known answers; see make_golden.py for where each comes from",
        # literals of the reference's own tests
        "mul1_known": {"0": 49896, "1": 14625, "7": 47511},           # src/core/format.zig:427-431
        "mcg_known": {"0": 0x3F60},                                     # src/core/format.zig:441-445
        "perm_known": {"0": 0, "1": 16, "4": 8},                       # src/core/format.zig:512-523
        "bit_end": {"64": {"0": 4}, "80": {"15": 80}, "36": {"0": 2, "3": 9}},  # src/core/format.zig:447-478
        "window_masks": {"16": 0xFFFF, "12": 0x0FFF, "8": 0x00FF},    # src/core/format.zig:447-478
        "partition_pins": {                                             # src/hip/plan.zig:206-215,366-371
            "rb_cap": [[5, 5, 5], [6, 5, 3], [16, 8, 8], [11, 8, 6]],
            "bt_for": [[1, 4], [5, 1]],
            "ks_for": [[2560, 640, 20]],
            "ks_gu_dn": [[2560, 640, 4, 2]],
        },
        # numpy restatements, whole tables by digest and a few entries in clear
        "mcg_table_sha256": hashlib.sha256(mcg.astype("<u2").tobytes()).hexdigest(),
        "mul1_table_sha256": hashlib.sha256(mul1.astype("<u2").tobytes()).hexdigest(),
        "mcg_samples": {str(c): int(mcg[c]) for c in (0, 1, 2, 255, 4096, 0x8000, 0xFFFF)},
        "mul1_samples": {str(c): int(mul1[c]) for c in (0, 1, 7, 255, 4096, 0x8000, 0xFFFF)},
        "tensor_core_perm": tensor_core_perm(),
        "tiles": tiles,
    }
    with open(os.path.join(HERE, "exl3_golden.json"), "w") as f:
        json.dump(golden, f, indent=1)
    print("wrote", os.path.join(HERE, "exl3_golden.json"))


if __name__ == "__main__":
    main()
