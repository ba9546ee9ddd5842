"""SwiGLU MLP host for the carved path: _SwiGLUMortar / _KwargSequential / _make_swiglu.

Interface mirror of morph/model/transformer.py:259-431.  Once gate_up and down are carved and ternary, the
forward is two HIP launches: gate_up with the SwiGLU (and the per-cluster router gates) fused into its
epilogue, then down.  Before carving the layers run their dense forward.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from .sparsity import MortarLinear



class _KwargSequential(nn.Sequential):
    """nn.Sequential that forwards **kwargs (iter_idx) to its first child; children keep indices "0"/"1"."""

    def forward(self, x, **kwargs):
        it = iter(self)
        x = next(it)(x, **kwargs)
        for m in it:
            x = m(x)
        return x

    def enable_routing(self, *args, **kwargs):
        return self[0].enable_routing(*args, **kwargs)

    @property
    def router(self):
        return getattr(self[0], "router", None)

    @property
    def d_ff(self):
        return self[0].d_ff


def _make_swiglu(d_model: int, d_ff: int, dropout: float) -> nn.Module:
    mlp: nn.Module = _SwiGLUMortar(d_model, d_ff)
    if dropout > 0:
        return _KwargSequential(mlp, nn.Dropout(dropout))
    return mlp


class _SwiGLUMortarFn(torch.autograd.Function):
    """The carved MLP as one differentiable op for QAT training: y = down(silu(gate) * up), gate_up kept for the
    backward.  Forward: SpMM, SwiGLU, SpMM.  Backward (reference: torch autograd over transformer.py:411-431 with the
    stk backward, custom_ops.py:99-136): dh through down's W^T pack, dW_down on the topology, the SwiGLU derivative in
    one launch, dx through gate_up's W^T pack, dW_gate_up on the topology."""

    @staticmethod
    def forward(ctx, x: Tensor, data_gu: Tensor, data_dn: Tensor, mlp: "_SwiGLUMortar") -> Tensor:
        cg, cd = mlp.gate_up._cms, mlp.down._cms
        cg.invalidate_pack(); cd.invalidate_pack()     # re-encode: .data writes do not advance the version counter
        gu = ops.spmm(x, cg.mortar_pack())
        h = ops.swiglu(gu)
        y = ops.spmm(h, cd.mortar_pack())
        ctx.mlp = mlp
        ctx.dtypes = (data_gu.dtype, data_dn.dtype)
        ctx.save_for_backward(x, gu, h)
        return y

    @staticmethod
    def backward(ctx, dy: Tensor):
        x, gu, h = ctx.saved_tensors
        cg, cd = ctx.mlp.gate_up._cms, ctx.mlp.down._cms
        dy = (dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)).contiguous()
        need_x, need_gu, need_dn = ctx.needs_input_grad[:3]
        d_dn = ops.sdd(dy, h, cd.mortar_pack()).to(ctx.dtypes[1]) if need_dn else None
        dx = d_gu = None
        if need_x or need_gu:
            dgu = ops.swiglu_backward(gu, ops.spmm(dy, cd.mortar_pack_t()))
            if need_gu:
                d_gu = ops.sdd(dgu, x, cg.mortar_pack()).to(ctx.dtypes[0])
            if need_x:
                dx = ops.spmm(dgu, cg.mortar_pack_t())
        return dx, d_gu, d_dn, None


class _SwiGLUMortar(nn.Module):
    def __init__(self, d_model: int, d_ff: int):
        super().__init__()
        self.gate_up = MortarLinear(d_model, d_ff * 2, bias=False, initial_density=1.0)
        self.down = MortarLinear(d_ff, d_model, bias=False, initial_density=1.0)
        self.d_model, self.d_ff = d_model, d_ff
        self.router: nn.Module | None = None
        self._last_aux_loss: Tensor | None = None
        self._aux_detach_input = True
        # Token lists + routed gate_up + masked down for prefill-sized routed calls.  Off by default: at 352 clusters of
        # one block-row, k = 88, 4096 tokens the list form measured 1.18 x the time of the plain step, while gates
        # multiplied in the gate_up epilogue cost the plain step plus the gates launch.  The list kernels stay as a
        # tested option for routers with few large clusters.
        self.route_skip = False

    def enable_routing(self, n_clusters: int = 16, activation_ratio: float = 0.5, aux_loss_coeff: float = 1e-2,
                       n_iters: int = 1, n_sub_keys: int = 0, detach_input: bool = True) -> None:
        """Attach an iteration-aware TileRouter over the d_ff hidden neuron bank (transformer.py:344-400)."""
        self._aux_detach_input = bool(detach_input)
        from .routing import TileRouter
        try:
            dev = next(self.down.parameters()).device
        except StopIteration:
            dev = next(self.down.buffers()).device
        self.router = TileRouter(n_tile_groups=n_clusters, d_model=self.d_model, activation_ratio=activation_ratio,
                                 n_sub_keys=n_sub_keys, aux_loss_coeff=aux_loss_coeff, n_iters=n_iters).to(dev)
        self.n_clusters = n_clusters
        base, rem = self.d_ff // n_clusters, self.d_ff % n_clusters
        sizes = torch.tensor([base + (1 if c < rem else 0) for c in range(n_clusters)])
        self.register_buffer("hidden_to_cluster", torch.repeat_interleave(torch.arange(n_clusters), sizes).to(dev))

    def _carved(self) -> bool:
        return self.gate_up._cms._mortar and self.down._cms._mortar

    def _wants_grad(self, x: Tensor) -> bool:
        """Autograd is recording and something upstream or the QAT block values need a gradient: the MLP then runs
        layer by layer (carved linear -> SwiGLU in torch -> carved linear) so that every step has a backward."""
        if not torch.is_grad_enabled():
            return False
        if x.requires_grad:
            return True
        return any(isinstance(getattr(m._cms, "mortar_data", None), torch.nn.Parameter) and m._cms.mortar_data.requires_grad
                   and "mortar_packed" not in m._cms._buffers for m in (self.gate_up, self.down))

    def forward(self, x: Tensor, iter_idx: int = 0, gates: Tensor | None = None, norm: tuple | None = None) -> Tensor:
        """x [..., d_model] -> [..., d_model].  ``gates`` overrides the router output (fp32 [N, n_clusters]);
        it exists so that a caller which already evaluated the router (or holds seeded logits) can feed it.
        ``norm`` = (weight or None, eps): x is the activation BEFORE the block's RMSNorm (norm_mlp) and the norm is
        applied here, inside the gate_up launch when the matrix allows it; same result as mlp(rmsnorm(x))."""
        train = self._carved() and self._wants_grad(x)
        if norm is not None:
            fused = (self._carved() and x.is_cuda and not train and (self.router is None or gates is not None)
                     and ops.norm_fusable(self.gate_up._cms.mortar_pack()))
            if not fused:
                nw, eps = norm
                if self._carved() and x.is_cuda and not train:
                    x = ops.rmsnorm(x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16), nw, eps)
                else:
                    xn = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)
                    x = xn * nw.to(x.dtype) if nw is not None else xn
                norm = None
            elif norm[0] is not None and norm[0].dtype != torch.bfloat16:
                norm = (norm[0].to(torch.bfloat16), norm[1])
        if (train and x.is_cuda and self.router is None and gates is None and norm is None
                and all(m._cms._values_ternary_mode and "mortar_packed" not in m._cms._buffers and m._cms.bias is None
                        for m in (self.gate_up, self.down))):
            lead = x.shape[:-1]
            x2 = x.reshape(-1, self.d_model)
            xb = x2 if x2.dtype == torch.bfloat16 else x2.to(torch.bfloat16)
            y = _SwiGLUMortarFn.apply(xb, self.gate_up._cms.mortar_data, self.down._cms.mortar_data, self)
            return (y if y.dtype == x.dtype else y.to(x.dtype)).reshape(*lead, self.d_model)
        if not self._carved() or train:
            gu = self.gate_up(x)
            gate, up = gu.chunk(2, dim=-1)
            h = F.silu(gate) * up
            if self.router is not None or gates is not None:
                if gates is None:
                    gates, aux = self.router(x.detach() if self._aux_detach_input else x, iter_idx=iter_idx)
                    self._last_aux_loss = aux
                g = gates.to(h.dtype).reshape(*h.shape[:-1], -1)
                ncl = g.shape[-1]
                if self.d_ff % ncl == 0:
                    h = (h.unflatten(-1, (ncl, self.d_ff // ncl)) * g.unsqueeze(-1)).flatten(-2)
                else:
                    h = h * g[..., self.hidden_to_cluster]
            return self.down(h)

        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.d_model)
        xb = x2 if x2.dtype == torch.bfloat16 else x2.to(torch.bfloat16)
        Wgu, Wdn = self.gate_up._cms.mortar_pack(), self.down._cms.mortar_pack()
        active = None
        if gates is None and self.router is not None:
            rx = x2.detach() if self._aux_detach_input else x2
            g3, aux = self.router(rx, iter_idx=iter_idx)
            self._last_aux_loss = aux
            gates = g3.detach().reshape(-1, g3.shape[-1]).float().contiguous()
            # the mask is derived below from the gates of THIS call (active = gates > 0, routing.py:258), never from
            # router state, which an earlier call of another shape may have left behind
        elif gates is not None:
            gates = gates.reshape(-1, gates.shape[-1]).float().contiguous()
        if gates is not None and self.d_ff % gates.shape[-1]:
            raise ValueError("the carved MLP needs equal-size clusters (d_ff % n_clusters == 0)")
        N = xb.shape[0]
        cs = self.d_ff // gates.shape[-1] if gates is not None else 0
        # decode-sized batches need no token lists: the gated gate_up kernel itself leaves out units whose cluster is
        # off for all tokens of its 4- or 16-token tile and stores their zeros
        tile = ops.route_tile(Wgu, N) if (gates is not None and self.route_skip and cs % 16 == 0 and N > ops.DECODE_MAX_ROWS) else 0
        if tile:
            if active is None:
                active = (gates > 0).to(torch.uint8)
            route = ops.remoe_route(active, tile)
            h = ops.gateup_swiglu(xb, Wgu, gates=gates, route=route, norm=norm)
            y = ops.spmm(h, Wdn, active=active)
        elif N > ops.DECODE_MAX_ROWS:
            y = ops.mlp(xb, Wgu, Wdn, gates=gates, norm=norm)      # hidden activations in the library's tile order
        else:
            h = ops.gateup_swiglu(xb, Wgu, gates=gates, norm=norm)
            y = ops.spmm(h, Wdn)
        if y.dtype != x.dtype:
            y = y.to(x.dtype)
        return y.reshape(*lead, self.d_model)
