"""stk_dds: the reference's sparse-backend operator signature (morph/sparse/stk/backend/custom_ops.py:35-56)
served by the HIP SpMM.  The MORTAR runtime executes ternary blocks, so ``data`` must be ternary-valued per
block (+-s_j or 0); the packed form is cached per data tensor."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops
from .deploy_quant import pack_ternary_codes
from .pack import MortarPack

_cache: dict = {}


def _pack_from_data(data: Tensor, offsets: Tensor, column_indices: Tensor, out_f: int, in_f: int) -> MortarPack:
    key = (data.data_ptr(), data._version, tuple(data.shape), out_f, in_f)
    hit = _cache.get(key)
    if hit is not None:
        return hit
    d = data.detach().float()
    if d.dim() != 3 or d.shape[1] != 16 or d.shape[2] != 16:
        raise ValueError(f"stk_dds: data must be [nnz, 16, 16] (carve(blocking=16)), got {tuple(data.shape)}")
    scale = d.abs().amax(dim=(1, 2))
    q = torch.sign(d)
    if not torch.equal(q * scale[:, None, None], d):
        raise ValueError("stk_dds: data is not ternary per block (+-s_j or 0); quantise it first")
    pack = MortarPack(pack_ternary_codes(q), scale, column_indices, offsets, out_f, in_f, data.device)
    if len(_cache) > 64:
        _cache.clear()
    _cache[key] = pack
    return pack


def stk_dds(lhs: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor, column_indices: Tensor,
            offsets_t: Tensor, column_indices_t: Tensor, block_offsets_t: Tensor,
            shape0: int, shape1: int, transpose_b: bool) -> Tensor:
    """transpose_b=True: stored BCSR matrix is (shape1, shape0); returns lhs @ W^T as a fresh [M, shape1]
    tensor of lhs.dtype.  Only the forward orientation (transpose_b=True) is on this path."""
    if not transpose_b:
        raise NotImplementedError("stk_dds(transpose_b=False) is the dX backward, outside the forward path")
    if row_indices.dtype != torch.int16 or column_indices.dtype != torch.int16:
        raise ValueError(f"Expected int16 row/column indices. Got {row_indices.dtype} / {column_indices.dtype}.")
    if offsets.dtype != torch.int32:
        raise ValueError(f"Expected int32 offsets. Got {offsets.dtype} offsets.")
    assert lhs.shape[1] == shape0, "incompatible dimensions"
    W = _pack_from_data(data, offsets, column_indices, shape1, shape0)
    x = lhs if lhs.dtype == torch.bfloat16 else lhs.to(torch.bfloat16)
    y = ops.spmm(x, W)
    return y if y.dtype == lhs.dtype else y.to(lhs.dtype)
