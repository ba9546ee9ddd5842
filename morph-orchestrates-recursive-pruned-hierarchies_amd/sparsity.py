"""MortarLinear: nn.Linear-shaped wrapper over CMSBlockLinear (reference: morph/model/sparsity.py:33-166)."""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor, nn

from .block_sparse import CMSBlockLinear


class MortarLinear(nn.Module):
    """Dense pre-carve (F.linear), MORTAR BCSR post-carve (HIP kernels).  Same constructor arguments,
    attributes (``_cms``, ``in_features``, ``out_features``, ``tile_size``) and methods as the reference."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, tile_size: int = 16,
                 initial_density: float = 1.0, score_ema_alpha: float = 0.95,
                 device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None) -> None:
        super().__init__()
        density = max(0.1, min(1.0, initial_density))
        self._cms = CMSBlockLinear(in_features=in_features, out_features=out_features, tile_size=tile_size,
                                   density=density, bias=bias, score_ema_alpha=score_ema_alpha,
                                   device=device, dtype=dtype)
        self.in_features, self.out_features, self.tile_size = in_features, out_features, tile_size

    @property
    def is_compact(self) -> bool:
        return not self._cms._dense_mode

    @property
    def bias(self) -> Optional[nn.Parameter]:
        return self._cms.bias

    def carve(self, blocking: int = 16) -> int:
        return self._cms.carve(blocking=blocking)

    def get_density(self) -> float:
        return self._cms.get_density()

    def forward(self, x: Tensor) -> Tensor:
        return self._cms(x)

    def extra_repr(self) -> str:
        mode = "mortar" if self.is_compact else "dense"
        return (f"in={self.in_features}, out={self.out_features}, tile={self.tile_size}, "
                f"density={self.get_density():.2f}, mode={mode}")
