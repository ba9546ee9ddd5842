"""stk_dds: the reference's sparse-backend operator signature (morph/sparse/stk/backend/custom_ops.py:35-56)
served by the HIP SpMM.  The MORTAR runtime executes ternary blocks, so ``data`` must be ternary-valued per
block (+-s_j or 0); the packed form is cached per data tensor."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops
from .pack import MortarPack

_cache: dict = {}


def _pack_from_data(data: Tensor, offsets: Tensor, column_indices: Tensor, out_f: int, in_f: int) -> MortarPack:
    """Pack of the stored matrix [out_f, in_f]: the topology is packed once per (offsets, column_indices) on the
    host, the values are ternarised and encoded on the device whenever ``data`` changed."""
    d = data.detach()
    if d.dim() != 3 or d.shape[1] != 16 or d.shape[2] != 16:
        raise ValueError(f"stk_dds: data must be [nnz, 16, 16] (carve(blocking=16)), got {tuple(data.shape)}")
    tkey = (offsets.data_ptr(), column_indices.data_ptr(), int(d.shape[0]), out_f, in_f, str(d.device))
    pack = _cache.get(tkey)
    if pack is None:
        if len(_cache) > 64:
            _cache.clear()
        pack = MortarPack(None, None, column_indices, offsets, out_f, in_f, d.device)
        pack._values_key = pack._t_values_key = None
        _cache[tkey] = pack
    vkey = (d.data_ptr(), d._version)
    if pack._values_key != vkey:
        df = d if d.dtype in (torch.bfloat16, torch.float32) else d.float()
        scale = df.abs().amax(dim=(1, 2)).float()
        if not torch.equal(torch.sign(df.float()) * scale[:, None, None], df.float()):
            raise ValueError("stk_dds: data is not ternary per block (+-s_j or 0); quantise it first")
        pack._scale = scale
        pack._values = df.contiguous()
        pack.requantize(pack._values, scale=scale, threshold=0.5, sync=False)
        pack._values_key = vkey
    return pack


def _transposed_pack(pack: MortarPack) -> MortarPack:
    t = pack.transposed()
    if pack._t_values_key != pack._values_key:
        t.requantize(pack._values, scale=pack._scale, threshold=0.5, transpose=True, sync=False)
        pack._t_values_key = pack._values_key
    return t


def stk_dds(lhs: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor, column_indices: Tensor,
            offsets_t: Tensor, column_indices_t: Tensor, block_offsets_t: Tensor,
            shape0: int, shape1: int, transpose_b: bool) -> Tensor:
    """transpose_b=True: the stored BCSR matrix is (shape1, shape0); returns lhs @ W^T as a fresh [M, shape1] tensor
    of lhs.dtype (the carved forward).  transpose_b=False: the stored matrix is (shape0, shape1); returns lhs @ W
    (the dX product), computed through the pack of W^T, whose topology is derived from offsets / column_indices
    (the *_t arguments carry the same information and are accepted for signature compatibility)."""
    if row_indices.dtype != torch.int16 or column_indices.dtype != torch.int16:
        raise ValueError(f"Expected int16 row/column indices. Got {row_indices.dtype} / {column_indices.dtype}.")
    if offsets.dtype != torch.int32:
        raise ValueError(f"Expected int32 offsets. Got {offsets.dtype} offsets.")
    assert lhs.shape[1] == shape0, "incompatible dimensions"
    if transpose_b:
        W = _pack_from_data(data, offsets, column_indices, shape1, shape0)
    else:
        W = _transposed_pack(_pack_from_data(data, offsets, column_indices, shape0, shape1))
    x = lhs if lhs.dtype == torch.bfloat16 else lhs.to(torch.bfloat16)
    y = ops.spmm(x, W)
    return y if y.dtype == lhs.dtype else y.to(lhs.dtype)
