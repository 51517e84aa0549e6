"""Loading an EXL3 pack for the quant table: the step before `table.matmul` / `table.swiglu`.

A pack is a directory with `config.json` and `*.safetensors`. Its config names the blocks this table is offered
(`trunk_quant` for the trunk's dense linears, `expert_quant` for the routed banks); the table claims and validates
each as the reference does (table/config.zig:54-85), then loads weights by the names the reference reads
(table/table.zig:124-174): a trunk linear is `<base>.weight` (trellis U16/I16 [in/16, out/16, n]), `<base>.scales`
(suh F16 [in]) and `<base>.biases` (svh F16 [out]); a bank is `<base>.trellis` (U16 [E, in/16, out/16, n]),
`<base>.suh`, `<base>.svh`. Tensors go to the device as stored: nothing is repacked or converted.
"""
from __future__ import annotations

import glob
import json
import os
from typing import Dict, Optional

import torch

from . import _lib, table


class Pack:
    def __init__(self, directory: str, device: str = "cuda", matrix_gate: bool = True):
        from safetensors import safe_open

        self.directory, self.device = directory, torch.device(device)
        with open(os.path.join(directory, "config.json")) as f:
            self.config_json = f.read()
        self.config = json.loads(self.config_json)
        self._files: Dict[str, str] = {}
        self._open = {}
        for path in sorted(glob.glob(os.path.join(directory, "*.safetensors"))):
            with safe_open(path, framework="pt", device="cpu") as f:
                for name in f.keys():
                    self._files[name] = path
        self._safe_open = safe_open
        # the blocks this table is offered, claimed and validated as the server's load preflight does
        self.blocks: Dict[str, Optional[_lib.Block]] = {}
        self.claims: Dict[str, str] = {}
        text = self.config.get("text_config") if isinstance(self.config.get("text_config"), dict) else {}
        for key in ("trunk_quant", "expert_quant"):
            block = self.config.get(key, text.get(key))
            if block is None:
                continue
            block_json = json.dumps(block)
            self.claims[key] = table.claims(block_json, self.config_json, matrix_gate)
            if self.claims[key] == "no":
                self.blocks[key] = None
                continue
            table.validate(block_json, self.config_json)  # raises table.Refused with the reference's reason
            self.blocks[key] = table.parse_block(block_json)

    def names(self):
        return self._files.keys()

    def _tensor(self, name: str):
        path = self._files.get(name)
        if path is None:
            return None
        with self._safe_open(path, framework="pt", device="cpu") as f:
            return f.get_tensor(name).to(self.device)

    def stored_bytes(self, base: str, leaves) -> int:
        total = 0
        for leaf in leaves:
            path = self._files.get(f"{base}.{leaf}")
            if path is None:
                continue
            with self._safe_open(path, framework="pt", device="cpu") as f:
                sl = f.get_slice(f"{base}.{leaf}")
                count = 1
                for d in sl.get_shape():
                    count *= d
                total += count * {"F32": 4, "I32": 4, "U32": 4}.get(sl.get_dtype(), 2)
        return total

    def linear(self, base: str, in_dim: int = 0) -> _lib.Weight:
        """A trunk linear under the pack's `trunk_quant` block (`load_tensor`)."""
        block = self.blocks.get("trunk_quant")
        if block is None:
            raise table.Refused(_lib.VERDICT_UNSUPPORTED, "turboexl3: the pack has no trunk_quant block this table claims")
        return table.load_tensor(block, self._tensor(f"{base}.weight"), self._tensor(f"{base}.scales"),
                                 self._tensor(f"{base}.biases"), in_dim)

    def bank(self, base: str, in_dim: int = 0) -> _lib.Weight:
        """One projection's routed bank under the pack's `expert_quant` block (`load_bank`)."""
        block = self.blocks.get("expert_quant")
        if block is None:
            raise table.Refused(_lib.VERDICT_UNSUPPORTED, "turboexl3: the pack has no expert_quant block this table claims")
        return table.load_bank(block, self._tensor(f"{base}.trellis"), self._tensor(f"{base}.suh"),
                               self._tensor(f"{base}.svh"), in_dim)

    def bill(self, key: str, base: str) -> int:
        """The block's bill for one weight: its stored bytes (table/config.zig:88-92)."""
        leaves = ("weight", "scales", "biases") if key == "trunk_quant" else ("trellis", "suh", "svh")
        return table.bill(json.dumps(self.config.get(key, {})), self.directory, self.stored_bytes(base, leaves))
