"""MORTAR sparse-MLP runtime for MI355X (gfx950): carved 16x16 BCSR ternary SpMM behind the reference's
MortarLinear / _SwiGLUMortar / stk_dds / mortar_gemv interfaces, served by hand-written HIP kernels."""
from . import _lib, ops, pack, synth                                   # noqa: F401
from .block_sparse import CMSBlockLinear                              # noqa: F401
from .deploy_quant import (pack_mortar_ternary, pack_ternary_codes, shrink_mlp_to_mortar_ternary,  # noqa: F401
                           unpack_ternary)
from .engine import MortarDecodeMLP, looped_core_forward, mortar_gemv, mortar_pack_strips  # noqa: F401
from .mlp import _KwargSequential, _make_swiglu, _SwiGLUMortar        # noqa: F401
from .pack import MortarPack                                          # noqa: F401
from .routing import TileRouter                                       # noqa: F401
from .sparsity import MortarLinear                                    # noqa: F401
from .stk import stk_dds, stk_sdd_at_b                                # noqa: F401

__all__ = ["CMSBlockLinear", "MortarLinear", "_SwiGLUMortar", "_KwargSequential", "_make_swiglu", "TileRouter",
           "MortarPack", "MortarDecodeMLP", "stk_dds", "stk_sdd_at_b", "mortar_gemv", "mortar_pack_strips", "looped_core_forward",
           "pack_mortar_ternary", "pack_ternary_codes", "unpack_ternary", "shrink_mlp_to_mortar_ternary",
           "ops", "pack", "synth"]
