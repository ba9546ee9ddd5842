"""TileRouter: PEER product-key + ReMoE ReLU gating over d_ff neuron clusters.

Interface mirror of the reference's morph/model/routing.py (same parameters, forward signature, outputs).
The gating tail (steps 5-8: k-th largest threshold, ReLU, normalise to sum k, active mask) runs in the HIP
kernel for inference.  For decode-sized calls (up to 64 rows) the front end (query projection, LayerNorm, sub-key
scores, product-key logits) runs in HIP as well, two launches in all; larger calls run the dense query projection as
a library GEMM through torch and everything behind it (LayerNorm to gates) in one HIP launch.
With autograd enabled the tail stays in differentiable torch ops.
"""
from __future__ import annotations

import math
from typing import Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops


def gates_from_logits(group_logits: Tensor, k: int) -> tuple[Tensor, Tensor]:
    """Inference tail on the device: (gates fp32 [N, n], active uint8 [N, n])."""
    return ops.remoe_gates(group_logits.float(), k)


class TileRouter(nn.Module):
    def __init__(self, n_tile_groups: int, d_model: int, activation_ratio: float = 0.5, n_sub_keys: int = 0,
                 aux_loss_coeff: float = 1e-2, n_iters: int = 1) -> None:
        super().__init__()
        self.n_tile_groups, self.d_model = n_tile_groups, d_model
        self.activation_ratio = activation_ratio
        self.activation_k = max(1, round(activation_ratio * n_tile_groups))
        self.aux_loss_coeff = aux_loss_coeff
        if n_sub_keys <= 0:
            n_sub_keys = max(4, math.ceil(math.sqrt(n_tile_groups)))
        self.n_sub_keys = n_sub_keys
        d_half = d_model // 2
        self.query_proj = nn.Linear(d_model, d_model, bias=False)
        self.sub_keys_a = nn.Parameter(torch.randn(n_sub_keys, d_half) * (d_half ** -0.5))
        self.sub_keys_b = nn.Parameter(torch.randn(n_sub_keys, d_half) * (d_half ** -0.5))
        self.group_bias = nn.Parameter(torch.zeros(n_tile_groups))
        self.n_iters = max(1, int(n_iters))
        self.iter_embed = nn.Parameter(torch.zeros(self.n_iters, d_model))
        self.query_norm = nn.LayerNorm(d_model)
        self.register_buffer("group_load_ema", torch.ones(n_tile_groups) / n_tile_groups)
        self._load_ema_alpha = 0.99
        self.last_active: Tensor | None = None      # uint8 [N, n] of the most recent forward / route call (diagnostics)

    def group_logits(self, x_flat: Tensor, iter_idx: int = 0) -> Tensor:
        """Steps 1-4 (reference routing.py:181-230): projected, normalised query -> product-key logits."""
        proj_dtype = self.query_proj.weight.dtype
        it = max(0, min(int(iter_idx), self.n_iters - 1))
        q = self.query_norm(self.query_proj(x_flat.to(proj_dtype)) + self.iter_embed[it].to(proj_dtype))
        d_half = self.d_model // 2
        sa = q[:, :d_half] @ self.sub_keys_a.T
        sb = q[:, d_half:] @ self.sub_keys_b.T
        n_products = self.n_sub_keys * self.n_sub_keys
        ps = (sa.unsqueeze(2) + sb.unsqueeze(1)).reshape(x_flat.shape[0], n_products)
        if n_products == self.n_tile_groups:
            return ps + self.group_bias.unsqueeze(0)
        if n_products >= self.n_tile_groups:
            top_scores, _ = ps.topk(self.n_tile_groups, dim=-1)
            return top_scores + self.group_bias.unsqueeze(0)
        idx = torch.arange(self.n_tile_groups, device=x_flat.device) % n_products
        return ps[:, idx] + self.group_bias.unsqueeze(0)

    def _fused_ok(self, x_flat: Tensor) -> bool:
        """Decode-sized inference calls on the GPU with fp32 router parameters go through the two-launch HIP router."""
        return (x_flat.is_cuda and 0 < x_flat.shape[0] <= ops.ROUTER_MAX_TOKENS and not torch.is_grad_enabled()
                and x_flat.dtype in (torch.bfloat16, torch.float32) and self.query_proj.weight.dtype == torch.float32
                and self.n_sub_keys * self.n_sub_keys <= 2048 and self.d_model % 8 == 0
                and self.n_tile_groups <= 1024)

    def _tail_ok(self, x_flat: Tensor) -> bool:
        """Inference calls of any size on the GPU with fp32 router parameters: library GEMM for the projection, then the
        one-launch tail."""
        return (x_flat.is_cuda and x_flat.shape[0] > 0 and not torch.is_grad_enabled()
                and x_flat.dtype in (torch.bfloat16, torch.float32) and self.query_proj.weight.dtype == torch.float32
                and self.n_sub_keys * self.n_sub_keys <= max(1024, self.n_tile_groups) and self.d_model % 8 == 0
                and self.d_model <= 8192 and self.n_tile_groups <= 1024)

    @torch.no_grad()
    def route(self, x_flat: Tensor, iter_idx: int = 0) -> Tuple[Tensor, Tensor]:
        """Inference-only routing of [N, d_model] rows: (gates fp32 [N, n], active uint8 [N, n]) and nothing else (no
        load statistics, no auxiliary loss), as the reference's decode engine calls its fused router
        (morph/kernels/triton/fused_router.py:100-140).  Two launches for decode-sized N; a library GEMM for the query
        projection plus one launch for everything behind it otherwise."""
        if self._fused_ok(x_flat):
            it = max(0, min(int(iter_idx), self.n_iters - 1))
            return ops.router_fused(x_flat, self.query_proj.weight, self.iter_embed[it], self.query_norm.weight,
                                    self.query_norm.bias, self.query_norm.eps, self.sub_keys_a, self.sub_keys_b,
                                    self.group_bias, self.activation_k)
        if self._tail_ok(x_flat):
            it = max(0, min(int(iter_idx), self.n_iters - 1))
            qv = F.linear(x_flat.float(), self.query_proj.weight)
            return ops.router_tail(qv, self.iter_embed[it], self.query_norm.weight, self.query_norm.bias,
                                   self.query_norm.eps, self.sub_keys_a, self.sub_keys_b, self.group_bias, self.activation_k)
        return gates_from_logits(self.group_logits(x_flat, iter_idx), self.activation_k)

    def forward(self, x: Tensor, iter_idx: int = 0) -> Tuple[Tensor, Tensor]:
        orig_shape = x.shape
        x_flat = x.reshape(-1, orig_shape[-1])
        k = self.activation_k
        if self._fused_ok(x_flat) or self._tail_ok(x_flat):
            gates, active = self.route(x_flat, iter_idx)
            self.last_active = active
            logits = None
        else:
            logits = self.group_logits(x_flat, iter_idx)
        if logits is None:
            pass
        elif torch.is_grad_enabled() and logits.requires_grad:
            if k < self.n_tile_groups:
                kth = logits.topk(k, dim=-1).values[:, -1:]
                gates = F.relu(logits - kth)
            else:
                gates = F.relu(logits)
            gates = gates * (k / gates.sum(dim=-1, keepdim=True).clamp(min=1e-6))
            active = (gates > 0)
            self.last_active = active.detach().to(torch.uint8)
        else:
            gates, active = gates_from_logits(logits, k)
            self.last_active = active
        with torch.no_grad():
            batch_load = active.float().reshape(-1, self.n_tile_groups).mean(0)
            self.group_load_ema.mul_(self._load_ema_alpha).add_(batch_load, alpha=1 - self._load_ema_alpha)
        aux_loss = self.aux_loss_coeff * gates.reshape(-1, self.n_tile_groups).mean(0).var()
        if len(orig_shape) == 3:
            gates = gates.reshape(orig_shape[0], orig_shape[1], self.n_tile_groups)
        return gates, aux_loss
