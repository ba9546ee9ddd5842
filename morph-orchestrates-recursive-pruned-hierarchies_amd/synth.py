"""Seeded synthetic inputs for the benchmark configurations (topology, ternary codes, scales, activations).

Draw order for one matrix, from numpy Generator(PCG64(seed)): (1) per-row block counts (Zipf variant only:
one permutation of the rows), (2) for each block-row in order, one permutation of the block-columns of which
the first count are kept and sorted, (3) all codes at once with P(-1, 0, +1) = (0.3, 0.4, 0.3), (4) all
scales at once, U(0.01, 0.1) fp32.  The reference's analogous builder draws randperm(C)[:k].sort() per row
(tile-prover/proofs/decode/gemv_bw_30b.py:124-165).
"""
from __future__ import annotations

import numpy as np
import torch

from .pack import BLK, MortarPack


def row_counts(Rb: int, Cb: int, density: float, rng: np.random.Generator, zipf_s: float | None = None) -> np.ndarray:
    if zipf_s is None:
        return np.full(Rb, max(1, int(round(density * Cb))), dtype=np.int64)
    rank = rng.permutation(Rb) + 1
    w = rank.astype(np.float64) ** (-zipf_s)
    frac = w / w.mean() * density
    for _ in range(50):                               # clip to [5 %, 60 %], rescale the unclipped rows to the mean
        frac = np.clip(frac, 0.05, 0.60)
        free = (frac > 0.05) & (frac < 0.60)
        gap = density * Rb - frac.sum()
        if abs(gap) < 1e-9 or not free.any():
            break
        frac[free] *= 1.0 + gap / frac[free].sum()
    return np.maximum(1, np.round(np.clip(frac, 0.05, 0.60) * Cb)).astype(np.int64)


def synth_matrix(out_features: int, in_features: int, density: float = 0.25, seed: int = 0,
                 zipf_s: float | None = None, per_tensor_scale: bool = False) -> dict:
    """One carved ternary matrix in the reference's carve layout (numpy arrays)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    Rb, Cb = out_features // BLK, in_features // BLK
    counts = row_counts(Rb, Cb, density, rng, zipf_s)
    cols = [np.sort(rng.permutation(Cb)[:c]) for c in counts]
    col_idx = np.concatenate(cols).astype(np.int16)
    row_idx = np.repeat(np.arange(Rb), counts).astype(np.int16)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    nnz = int(offsets[-1])
    codes = rng.choice(np.array([-1, 0, 1], dtype=np.int8), size=(nnz, BLK, BLK), p=[0.3, 0.4, 0.3])
    scales = rng.uniform(0.01, 0.1, size=nnz).astype(np.float32)
    if per_tensor_scale:
        scales = scales[:1].copy()
    return dict(codes=codes, scales=scales, col_idx=col_idx, row_idx=row_idx, offsets=offsets,
                shape=(out_features, in_features))


def synth_x(M: int, d: int, seed: int = 0) -> np.ndarray:
    """Activations N(0,1) rounded to bf16, returned as float32 (bf16-representable values)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    x = rng.standard_normal((M, d), dtype=np.float32)
    return torch.from_numpy(x).to(torch.bfloat16).float().numpy()


def synth_logits(M: int, n: int, seed: int = 0) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((M, n), dtype=np.float32)


def flat_pack(codes: np.ndarray) -> np.ndarray:
    """int8 codes -> the reference's flat 2-bit pack (4 codes per byte, stored value code + 1)."""
    u = (codes.reshape(-1, 4).astype(np.int16) + 1).astype(np.uint8)
    return (u[:, 0] | (u[:, 1] << 2) | (u[:, 2] << 4) | (u[:, 3] << 6)).astype(np.uint8)


def to_pack(mat: dict, device, prefill_stream: bool = True, scale_after_sum: bool = True) -> MortarPack:
    out_f, in_f = mat["shape"]
    return MortarPack(flat_pack(mat["codes"]), mat["scales"], mat["col_idx"], mat["offsets"], out_f, in_f, device,
                      prefill_stream=prefill_stream, scale_after_sum=scale_after_sum)


def synth_mlp(d_model: int, d_ff: int, density: float = 0.25, seed: int = 0, zipf_s: float | None = None) -> dict:
    """gate_up [2*d_ff, d_model] (gate rows then up rows) and down [d_model, d_ff]."""
    return dict(gate_up=synth_matrix(2 * d_ff, d_model, density, seed * 2 + 1, zipf_s),
                down=synth_matrix(d_model, d_ff, density, seed * 2 + 2, zipf_s), d_model=d_model, d_ff=d_ff)


def carved_state(mat: dict, prefix: str = "") -> dict:
    """state_dict entries of a packed carved layer (the reference's key set) for one synthetic matrix."""
    from .block_sparse import _stk_transpose
    rows, cols = torch.from_numpy(mat["row_idx"]), torch.from_numpy(mat["col_idx"])
    offs = torch.from_numpy(mat["offsets"])
    ct, ot, bt = _stk_transpose(mat["shape"], torch.empty(0, BLK, BLK), rows, cols, offs)
    scales = torch.from_numpy(mat["scales"])
    return {prefix + "mortar_packed": torch.from_numpy(flat_pack(mat["codes"])),
            prefix + "mortar_scale": scales if scales.numel() > 1 else scales.reshape(()),
            prefix + "mortar_row_indices": rows, prefix + "mortar_column_indices": cols,
            prefix + "mortar_offsets": offs, prefix + "mortar_column_indices_t": ct,
            prefix + "mortar_offsets_t": ot, prefix + "mortar_block_offsets_t": bt,
            prefix + "mortar_ternary": torch.tensor([0.0, 0.5])}


def qat_state(mat: dict, prefix: str = "", seed: int = 0) -> dict:
    """state_dict entries of a carved layer in values-ternary QAT (bf16 mortar_data, not packed) on a synthetic
    topology: smooth values N(0, 0.05), the reference's key set (block_sparse.py:783-799)."""
    from .block_sparse import _stk_transpose
    rows, cols = torch.from_numpy(mat["row_idx"]), torch.from_numpy(mat["col_idx"])
    offs = torch.from_numpy(mat["offsets"])
    ct, ot, bt = _stk_transpose(mat["shape"], torch.empty(0, BLK, BLK), rows, cols, offs)
    g = torch.Generator().manual_seed(seed)
    data = (torch.randn(rows.numel(), BLK, BLK, generator=g) * 0.05).to(torch.bfloat16)
    return {prefix + "mortar_data": data, prefix + "mortar_row_indices": rows, prefix + "mortar_column_indices": cols,
            prefix + "mortar_offsets": offs, prefix + "mortar_column_indices_t": ct, prefix + "mortar_offsets_t": ot,
            prefix + "mortar_block_offsets_t": bt, prefix + "mortar_ternary": torch.tensor([1.0, 0.5])}


def qat_mlp_module(spec: dict, device, seed: int = 0):
    """A carved _SwiGLUMortar in values-ternary QAT (trainable bf16 block values) over the synthetic topologies."""
    from .mlp import _SwiGLUMortar
    with torch.device("meta"):
        mlp = _SwiGLUMortar(spec["d_model"], spec["d_ff"])
    mlp = mlp.to_empty(device="cpu")
    sd = {**qat_state(spec["gate_up"], "gate_up._cms.", seed), **qat_state(spec["down"], "down._cms.", seed + 1)}
    mlp.load_state_dict(sd, strict=True)
    return mlp.to(device)


def mlp_module(spec: dict, device):
    """A carved, packed _SwiGLUMortar holding the synthetic matrices, loaded through load_state_dict."""
    from .mlp import _SwiGLUMortar
    with torch.device("meta"):
        mlp = _SwiGLUMortar(spec["d_model"], spec["d_ff"])
    mlp = mlp.to_empty(device="cpu")
    sd = {**carved_state(spec["gate_up"], "gate_up._cms."), **carved_state(spec["down"], "down._cms.")}
    mlp.load_state_dict(sd, strict=True)
    return mlp.to(device)
