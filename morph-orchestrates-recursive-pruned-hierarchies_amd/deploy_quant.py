"""Ternary quantisation and 2-bit packing of carved blocks: host-side mirror of the MLP subset of the
reference's morph/inference/deploy_quant.py (same names, argument meaning and results)."""
from __future__ import annotations

import torch
from torch import Tensor, nn

__all__ = ["pack_ternary_codes", "unpack_ternary", "_ternary_quantize", "_ternary_quantize_per_block",
           "pack_mortar_ternary", "shrink_mlp_to_mortar_ternary"]

_CODES_PER_BYTE = 4
_PLACE = (1, 4, 16, 64)          # value of a code in slot 0..3 of its byte (2 bits each, slot 0 lowest)


def pack_ternary_codes(q: Tensor) -> Tensor:
    """{-1,0,+1} -> uint8, 4 codes per byte: byte = sum of (code + 1) * 4**slot over its four slots, flat order, the tail
    padded with stored value 0.  Same bytes as the reference's packer (deploy_quant.py:56-71)."""
    stored = q.reshape(-1).to(torch.int32) + 1
    n_bytes = -(-stored.numel() // _CODES_PER_BYTE)
    slots = stored.new_zeros(n_bytes * _CODES_PER_BYTE)
    slots[:stored.numel()] = stored
    place = torch.tensor(_PLACE, dtype=torch.int32, device=stored.device)
    return (slots.view(n_bytes, _CODES_PER_BYTE) * place).sum(dim=1).to(torch.uint8)


def unpack_ternary(packed: Tensor, numel: int, dtype: torch.dtype) -> Tensor:
    """The first ``numel`` codes of a pack_ternary_codes buffer as {-1,0,+1} in ``dtype`` (deploy_quant.py:74-78)."""
    b = packed.reshape(-1).to(torch.int32)
    stored = torch.stack([(b // p) % 4 for p in _PLACE], dim=1).reshape(-1)[:numel]
    return stored.to(dtype) - 1.0


def _ternary_codes(w: Tensor, scale: Tensor, threshold: float) -> Tensor:
    """sign(w / scale) where |w / scale| exceeds the threshold, else 0 (the quotient is formed first, as the reference
    does, so that values at the threshold round the same way)."""
    ratio = w / scale
    return torch.where(ratio.abs() > threshold, torch.sign(ratio), torch.zeros_like(ratio)).to(torch.int8)


def _ternary_quantize(w: Tensor, threshold: float = 0.5) -> tuple[Tensor, Tensor]:
    """Per-tensor symmetric ternary: scale = mean|w| (at least 1e-8), codes as _ternary_codes.
    Reference: deploy_quant.py:81-95; block_sparse.py:909-919."""
    w32 = w.detach().float()
    scale = w32.abs().mean().clamp(min=1e-8)
    return _ternary_codes(w32, scale, threshold), scale


def _ternary_quantize_per_block(w: Tensor, threshold: float = 0.5) -> tuple[Tensor, Tensor]:
    """The same rule with one scale per [blk, blk] block (mean|w| per block, at least 1e-6), the per-tile form
    of block_sparse.py:341-349,393-401 applied to carved blocks.  w [nnz, blk, blk] -> (codes, scale [nnz])."""
    w32 = w.detach().float()
    scale = w32.abs().mean(dim=(1, 2)).clamp(min=1e-6)
    return _ternary_codes(w32, scale[:, None, None], threshold), scale


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
