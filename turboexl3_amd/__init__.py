"""turboexl3's EXL3 projection engine for MI355X (gfx950): hand-written HIP kernels behind a C ABI, with the
reference's module entry points mirrored over torch device tensors."""
from .api import (MCG, MUL1, Bank, Decode, Proj, T3Error, configure, dequant, linear, linear_chain, moe, moe_clamped,
                  moe_shared_expert, moe_with_shared, release_engines)

__all__ = ["MCG", "MUL1", "Bank", "Decode", "Proj", "T3Error", "configure", "dequant", "linear", "linear_chain",
           "moe", "moe_clamped", "moe_shared_expert", "moe_with_shared", "release_engines"]
