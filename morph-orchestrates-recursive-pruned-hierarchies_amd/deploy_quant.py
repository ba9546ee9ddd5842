"""Ternary quantisation and 2-bit packing of carved blocks: host-side mirror of the MLP subset of the
reference's morph/inference/deploy_quant.py (same names, argument meaning and results)."""
from __future__ import annotations

import torch
from torch import Tensor, nn

__all__ = ["pack_ternary_codes", "unpack_ternary", "_ternary_quantize", "_ternary_quantize_per_block",
           "pack_mortar_ternary", "shrink_mlp_to_mortar_ternary"]

_SHIFTS = torch.tensor([0, 2, 4, 6], dtype=torch.uint8)


def pack_ternary_codes(q: Tensor) -> Tensor:
    """{-1,0,+1} -> uint8, 4 codes/byte, stored value = code + 1, little-endian in the byte, length padded
    to a multiple of 4 with zeros.  Reference: deploy_quant.py:56-71."""
    flat = q.reshape(-1)
    pad = (-flat.numel()) % 4
    u = (flat.to(torch.int16) + 1).to(torch.uint8)
    if pad:
        u = torch.cat([u, torch.zeros(pad, dtype=torch.uint8, device=u.device)])
    u = u.view(-1, 4)
    return (u[:, 0] | (u[:, 1] << 2) | (u[:, 2] << 4) | (u[:, 3] << 6)).contiguous()


def unpack_ternary(packed: Tensor, numel: int, dtype: torch.dtype) -> Tensor:
    """Inverse of pack_ternary_codes.  Reference: deploy_quant.py:74-78."""
    u = (packed.unsqueeze(-1) >> _SHIFTS.to(packed.device)) & 3
    return u.reshape(-1)[:numel].to(dtype) - 1.0


def _ternary_quantize(w: Tensor, threshold: float = 0.5) -> tuple[Tensor, Tensor]:
    """Per-tensor symmetric ternary: scale = mean|w| (clamp 1e-8), q = sign(w/s) * (|w/s| > threshold).
    Reference: deploy_quant.py:81-95; block_sparse.py:909-919."""
    wf = w.detach().float()
    scale = wf.abs().mean().clamp(min=1e-8)
    wn = wf / scale
    q = (torch.sign(wn) * (wn.abs() > threshold)).to(torch.int8)
    return q, scale


def _ternary_quantize_per_block(w: Tensor, threshold: float = 0.5) -> tuple[Tensor, Tensor]:
    """The same rule with one scale per [blk, blk] block (mean|w| per block, clamp 1e-6), the per-tile form
    of block_sparse.py:341-349,393-401 applied to carved blocks.  w [nnz, blk, blk] -> (codes, scale [nnz])."""
    wf = w.detach().float()
    scale = wf.abs().mean(dim=(1, 2)).clamp(min=1e-6)
    wn = wf / scale[:, None, None]
    q = (torch.sign(wn) * (wn.abs() > threshold)).to(torch.int8)
    return q, scale


def pack_mortar_ternary(cms: nn.Module, threshold: float = 0.5, per_block: bool = False) -> dict:
    """Ternarise + 2-bit-pack a carved CMSBlockLinear's mortar_data IN PLACE (reference:
    deploy_quant.py:344-374).  Registers ``mortar_packed`` (uint8) and ``mortar_scale`` (fp32 scalar, or
    [nnz] with per_block=True), sets ``_packed_shape`` / ``_packed_numel`` and drops the bf16 parameter."""
    assert getattr(cms, "_mortar", False), "pack_mortar_ternary requires a carved layer"
    assert not getattr(cms, "_values_ternary_mode", False), \
        "pack bakes the ternary snap; values-ternary STE must be OFF"
    data = cms.mortar_data.data
    shape = tuple(data.shape)
    q, scale = (_ternary_quantize_per_block if per_block else _ternary_quantize)(data, threshold)
    packed = pack_ternary_codes(q)
    del cms._parameters["mortar_data"]
    cms.register_buffer("mortar_packed", packed)
    cms.register_buffer("mortar_scale", scale)
    cms._packed_shape = shape
    cms._packed_numel = shape[0] * shape[1] * shape[2]
    cms._pack = None
    nz = int(q.ne(0).sum().item())
    return {"nnz_blocks": shape[0], "packed_bytes": packed.numel(),
            "scale": float(scale.float().mean()), "nonzero_code_frac": nz / max(1, q.numel())}


def shrink_mlp_to_mortar_ternary(bel, target_density: float = 0.25, blocking: int = 16, threshold: float = 0.5,
                                 generator: torch.Generator | None = None, per_block: bool = False) -> dict:
    """Systems-test pipeline for ONE MortarLinear, in place: uniform-random block saliency -> keep the
    top target_density of blocks (at least one per block-row) -> carve(blocking) -> ternary 2-bit pack.
    Reference: deploy_quant.py:400-428 (whose prune step lives in the out-of-scope pruning code; the
    selection rule -- global top fraction with a one-per-row floor -- follows block_sparse.py:664-712)."""
    cms = bel._cms
    Rb, Cb = cms.out_features // blocking, cms.in_features // blocking
    score = torch.rand((Rb, Cb), generator=generator)
    keep = max(Rb, int(round(target_density * Rb * Cb)))
    thr = torch.topk(score.flatten(), keep).values[-1]
    mask = score >= thr
    mask[torch.arange(Rb), score.argmax(dim=1)] = True
    cms.set_block_mask(mask, blocking)
    nnz = cms.carve(blocking=blocking)
    info = pack_mortar_ternary(cms, threshold, per_block=per_block)
    info.update(block_density=nnz / (Rb * Cb), nnz=nnz)
    return info
