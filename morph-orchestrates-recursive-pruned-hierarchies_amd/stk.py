"""stk_dds / stk_sdd_at_b: the reference's sparse-backend operators (morph/sparse/stk/backend/custom_ops.py:35-136)
served by the HIP kernels.  The MORTAR runtime executes ternary blocks, so ``data`` must be ternary-valued per
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


def _check_meta(offsets: Tensor, row_indices: Tensor, column_indices: Tensor) -> None:
    if row_indices.dtype != torch.int16 or column_indices.dtype != torch.int16:
        raise ValueError(f"Expected int16 row/column indices. Got {row_indices.dtype} / {column_indices.dtype}.")
    if offsets.dtype != torch.int32:
        raise ValueError(f"Expected int32 offsets. Got {offsets.dtype} offsets.")


@torch.library.custom_op("mortar_amd::dds", mutates_args=(), device_types="cuda")
def stk_dds(lhs: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor, column_indices: Tensor,
            offsets_t: Tensor, column_indices_t: Tensor, block_offsets_t: Tensor,
            shape0: int, shape1: int, transpose_b: bool) -> Tensor:
    """transpose_b=True: the stored BCSR matrix is (shape1, shape0); returns lhs @ W^T as a fresh [M, shape1] tensor
    of lhs.dtype (the carved forward).  transpose_b=False: the stored matrix is (shape0, shape1); returns lhs @ W
    (the dX product), computed through the pack of W^T, whose topology is derived from offsets / column_indices
    (the *_t arguments carry the same information and are accepted for signature compatibility).  Registered as a
    torch custom op with a fake implementation and the reference's backward (custom_ops.py:59-136)."""
    _check_meta(offsets, row_indices, column_indices)
    assert lhs.shape[1] == shape0, "incompatible dimensions"
    if transpose_b:
        W = _pack_from_data(data, offsets, column_indices, shape1, shape0)
    else:
        W = _transposed_pack(_pack_from_data(data, offsets, column_indices, shape0, shape1))
    x = lhs if lhs.dtype == torch.bfloat16 else lhs.to(torch.bfloat16)
    y = ops.spmm(x, W)
    return y if y.dtype == lhs.dtype else y.to(lhs.dtype)


@stk_dds.register_fake
def _stk_dds_fake(lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
                  shape0, shape1, transpose_b):
    return lhs.new_empty((lhs.size(0), shape1))


@torch.library.custom_op("mortar_amd::sdd_at_b", mutates_args=(), device_types="cuda")
def stk_sdd_at_b(a: Tensor, b: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor,
                 column_indices: Tensor) -> Tensor:
    """a^T @ b restricted to the topology of ``data`` ([nnz, 16, 16], values never read): the dW product
    (reference: custom_ops.py:78-96).  a [M, rows*16], b [M, cols*16]; result in a.dtype."""
    _check_meta(offsets, row_indices, column_indices)
    if data.dim() != 3 or data.shape[1] != 16 or data.shape[2] != 16:
        raise ValueError(f"stk_sdd_at_b: data must be [nnz, 16, 16], got {tuple(data.shape)}")
    tkey = (offsets.data_ptr(), column_indices.data_ptr(), int(data.shape[0]), a.shape[1], b.shape[1], str(a.device))
    W = _cache.get(tkey)
    if W is None:
        if len(_cache) > 64:
            _cache.clear()
        W = MortarPack(None, None, column_indices, offsets, a.shape[1], b.shape[1], a.device)
        W._values_key = W._t_values_key = None
        _cache[tkey] = W
    ab = a if a.dtype == torch.bfloat16 else a.to(torch.bfloat16)
    bb = b if b.dtype == torch.bfloat16 else b.to(torch.bfloat16)
    out = ops.sdd(ab, bb, W)
    return out if out.dtype == a.dtype else out.to(a.dtype)


@stk_sdd_at_b.register_fake
def _stk_sdd_fake(a, b, data, offsets, row_indices, column_indices):
    return a.new_empty(data.shape)


def _dds_setup_context(ctx, inputs, output):
    (lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
     shape0, shape1, transpose_b) = inputs
    ctx.save_for_backward(lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t)
    ctx.shape0, ctx.shape1, ctx.transpose_b = shape0, shape1, transpose_b


def _dds_backward(ctx, grad):
    """dlhs = grad @ (W if transpose_b else W^T): another dds; ddata = (grad^T @ lhs if transpose_b else lhs^T @ grad)
    on the topology: sdd (reference: custom_ops.py:99-136)."""
    lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t = ctx.saved_tensors
    dy = grad if grad.is_contiguous() else grad.contiguous()
    dlhs = ddata = None
    if ctx.needs_input_grad[0]:
        dlhs = stk_dds(dy, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
                       ctx.shape1, ctx.shape0, not ctx.transpose_b)
    if ctx.needs_input_grad[1]:
        a, b = (dy, lhs) if ctx.transpose_b else (lhs, dy)
        ddata = stk_sdd_at_b(a, b, data, offsets, row_indices, column_indices)
        if ddata.dtype != data.dtype:
            ddata = ddata.to(data.dtype)
    return (dlhs, ddata, None, None, None, None, None, None, None, None, None)


torch.library.register_autograd("mortar_amd::dds", _dds_backward, setup_context=_dds_setup_context)
