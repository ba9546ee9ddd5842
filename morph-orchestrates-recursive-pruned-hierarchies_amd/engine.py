"""Decode-side callers of the carved MLP: the reference engine's MLP subset
(morph/inference/engine.py:307-332,367-431,936-994) and its kernel entry points
(mortar_pack_strips / mortar_gemv, morph/kernels/triton/fused_decode_step.py:1465-1547)."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops
from .pack import MortarPack


def mortar_pack_strips(cms) -> MortarPack:
    """One-time engine pack of a pack_mortar_ternary'd CMSBlockLinear.  The reference returns the tuple
    (strips, col_idx, offsets, scale, out_features, ent, nspl_max, cnts); here the device format and the
    work lists live in one MortarPack (``.codes``, ``.col``, ``.row_ptr``, ``.sdup``, ``.out_features``,
    ``.worklist(...)``)."""
    return cms.mortar_pack()


def mortar_gemv(x: Tensor, pack: MortarPack, swiglu_x: bool = False, swiglu_out: bool = False,
                row_act: Tensor | None = None, col_act: Tensor | None = None, gates: Tensor | None = None,
                cluster_size: int = 0, flags_from_gates: bool = True) -> Tensor:
    """x [B, I] row-contiguous -> [B, O], or [B, O/2] = silu(g)*u with swiglu_out (the gate_up call); with swiglu_x,
    x is the packed gate_up output [B, 2I] and h = silu(g)*u is computed on load (the reference's down call form).
    Same keywords as the reference (fused_decode_step.py:1502-1509).  float32 input runs the reference engine's
    arithmetic (exact products, fp32 sums, fp32 scale after the block sum, fp32 out); bfloat16 input runs the bf16
    activation path of this runtime (swiglu_x there goes through the fp32 kernel and is rounded to bf16 at the end).
    row_act / col_act are per-stream flags as in the reference's kernel; ``flags_from_gates`` (see ops.gemv): they are
    route_flags of the same step's gates, which is how the reference engine calls (engine.py:984-994)."""
    if gates is not None and cluster_size and (pack.out_features // 2) // gates.shape[-1] != cluster_size:
        raise ValueError("cluster_size does not match d_ff / n_clusters")
    if x.dtype == torch.float32 or swiglu_x:
        y = ops.gemv_f32(x.float(), pack, swiglu_x=swiglu_x, swiglu_out=swiglu_out, gates=gates, row_act=row_act, col_act=col_act)
        return y if x.dtype == torch.float32 else y.to(x.dtype)
    return ops.gemv(x, pack, swiglu_out=swiglu_out, gates=gates, row_act=row_act, col_act=col_act, flags_from_gates=flags_from_gates)


class MortarDecodeMLP:
    """The engine's ``_mlp_fn`` MORTAR branch for one block: rmsnorm -> [router gates -> gather flags] ->
    gate_up GEMV with fused SwiGLU/gates -> down GEMV.  Packs are built once at construction."""

    def __init__(self, mlp, norm_weight: Tensor | None = None, eps: float = 1e-6, iter_idx: int = 0):
        self.mlp = mlp
        self.Mgu = mortar_pack_strips(mlp.gate_up._cms)
        self.Mdown = mortar_pack_strips(mlp.down._cms)
        self.norm_weight, self.eps, self.iter_idx = norm_weight, eps, iter_idx
        self.d_ff = mlp.d_ff

    @torch.no_grad()
    def __call__(self, x: Tensor, gates: Tensor | None = None) -> Tensor:
        B = x.shape[0]
        rt = getattr(self.mlp, "router", None)
        if (gates is not None or rt is None) and ops.norm_fusable(self.Mgu):
            # no router to feed: the norm rides on the gate_up launch (the reference folds it into its dense
            # ternary GEMV the same way, fused_decode_step.py X_MODE = 1)
            return self.mlp(x.reshape(B, -1).to(torch.bfloat16), iter_idx=self.iter_idx, gates=gates,
                            norm=(self.norm_weight, self.eps)).view(B, 1, -1)
        xn = ops.rmsnorm(x.reshape(B, -1).to(torch.bfloat16), self.norm_weight, self.eps)
        if gates is None and rt is not None:
            gates, _ = rt.route(xn, self.iter_idx)
        # the gated gate_up kernel leaves out the units whose cluster is off for every stream of its tile (and stores
        # their zeros), so `down` reads the hidden activations of inactive clusters as zero without a mask
        h = ops.gateup_swiglu(xn, self.Mgu, gates=gates.contiguous() if gates is not None else None)
        return ops.spmm(h, self.Mdown).view(B, 1, -1)


@torch.no_grad()
def looped_core_forward(mlps, x: Tensor, n_iters: int, norm_weights=None, eps: float = 1e-6, observer=None) -> Tensor:
    """Core-loop call pattern (morph/model/transformer.py:685-728,1146-1169) reduced to the MLP path:
    n_iters passes over the shared blocks, the same weights every pass, iter_idx = t forwarded to each MLP,
    activations RMS-normalised before every MLP (mhc.py:249-250).  ``observer(t, i, x_in, x_out)``, when given, is
    called after every MLP call with its input (before the norm) and output (diagnostics, the reference's
    ``_capture_traj``)."""
    for t in range(n_iters):
        for i, m in enumerate(mlps):
            w = norm_weights[i] if norm_weights is not None else None
            y = m(x, iter_idx=t, norm=(w, eps))
            if observer is not None:
                observer(t, i, x, y)
            x = y
    return x
