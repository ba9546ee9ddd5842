"""stk_dds / stk_sdd_at_b: the reference's sparse-backend operators (morph/sparse/stk/backend/custom_ops.py:35-136) served
by the HIP kernels.

``stk_dds`` multiplies whatever bf16 values ``data`` holds, as the reference's operator does (the product over stored
block values, ``ops.dds_values``).  ``stk_dds_ternary`` is the fast form for data that is ternary per block (0 or +-s_j,
what ``CMSBlockLinear._mortar_effective_data`` yields in values-ternary mode): the values are encoded on the device into
the 2- / 4-bit streams of the ternary kernels at every call, and data that is not ternary makes the result NaN."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops
from .pack import BcsrTopology, MortarPack

_cache: dict = {}
_tcache: dict = {}


def _key(offsets: Tensor, column_indices: Tensor, nnz: int, out_f: int, in_f: int, device):
    return (offsets.data_ptr(), offsets._version, column_indices.data_ptr(), column_indices._version, nnz, out_f, in_f, str(device))


def _bcsr(offsets: Tensor, column_indices: Tensor, nnz: int, out_f: int, in_f: int, device) -> BcsrTopology:
    """The index arrays of a topology on the device, built once per (offsets, column_indices) storage.  The entry keeps the
    two index tensors alive, so their addresses cannot be handed to other tensors while it is cached."""
    k = _key(offsets, column_indices, nnz, out_f, in_f, device)
    t = _tcache.get(k)
    if t is None:
        if len(_tcache) > 64:
            _tcache.clear()
        t = BcsrTopology(offsets, column_indices, out_f, in_f, device)
        t._keepalive = (offsets, column_indices)
        _tcache[k] = t
    return t


def _topology(offsets: Tensor, column_indices: Tensor, nnz: int, out_f: int, in_f: int, device) -> MortarPack:
    """The ternary pack of a topology (all-zero values), built once per (offsets, column_indices) storage."""
    tkey = _key(offsets, column_indices, nnz, out_f, in_f, device)
    pack = _cache.get(tkey)
    if pack is None:
        if len(_cache) > 64:
            stk_check()                      # a pending error of a pack about to be dropped is raised, not lost
            _cache.clear()
        pack = MortarPack(None, None, column_indices, offsets, out_f, in_f, device)
        pack._keepalive = (offsets, column_indices)
        _cache[tkey] = pack
    return pack


# A bf16 cast of +-s (1 + fp32 rounding) may land one bf16 step beside bf16(s): accepted as ternary.
_TERNARY_TOL = 2.0 ** -7


def _pack_from_data(data: Tensor, offsets: Tensor, column_indices: Tensor, out_f: int, in_f: int,
                    transposed: bool = False) -> MortarPack:
    """Pack of the stored matrix [out_f, in_f] (or of its transpose) for the ternary kernels: the topology is packed once on
    the host, the values are encoded on the device on EVERY call (no host synchronisation), so a data tensor that changed
    - in place or by being replaced at the same address - is always honoured.  The encode kernel checks that every value
    is 0 or +-s_j (s_j = the block's largest magnitude) and raises a flag on the device otherwise.  The first call on a
    topology waits for that flag; later calls read it without waiting, so the ValueError comes from the first call that
    finds the flag on the host (at the latest from ``stk_check()``) -- but the product of the offending call itself is
    already unusable: ``poison_on_status`` is enqueued behind it and turns the whole result into NaN on the device when
    the flag is set.  Values within 2^-7 of 0 or of +-s_j (relative to s_j) count as ternary: a bf16 cast of an fp32 +-s
    may land one bf16 step beside bf16(s)."""
    d = data.detach()
    if d.dim() != 3 or d.shape[1] != 16 or d.shape[2] != 16:
        raise ValueError(f"stk_dds_ternary: data must be [nnz, 16, 16] (carve(blocking=16)), got {tuple(data.shape)}")
    pack = _topology(offsets, column_indices, int(d.shape[0]), out_f, in_f, d.device)
    target = pack.transposed() if transposed else pack
    msg = target.poll_status()
    if msg is not None:
        raise ValueError("stk_dds_ternary (an earlier call): " + msg)
    df = (d if d.dtype in (torch.bfloat16, torch.float32) else d.float()).contiguous()
    scale = df.abs().amax(dim=(1, 2)).float()
    first = getattr(target, "_stk_checked", None) is None
    target.requantize(df, scale=scale, threshold=0.5, transpose=transposed, sync=False, ternary_tol=_TERNARY_TOL)
    if first:
        try:
            target.raise_status()
        except ValueError as e:
            raise ValueError("stk_dds_ternary: " + str(e).split(": ", 1)[-1]) from None
        target._stk_checked = True
    return target


def stk_check() -> None:
    """Waits for the device and raises ValueError if any stk_dds_ternary call so far was handed data that is not ternary
    per block.  Calls report such an error themselves once the device flag has reached the host; this is the synchronous
    form for the end of a step or a test."""
    for pack in list(_cache.values()):
        for t in (pack, pack._transposed):
            if t is not None:
                try:
                    t.raise_status()
                except ValueError as e:
                    raise ValueError("stk_dds_ternary: " + str(e).split(": ", 1)[-1]) from None


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
    (the dX product) through the transposed topology, which is derived from offsets / column_indices (the *_t arguments
    carry the same information and are accepted for signature compatibility).  Any block values: both operands are taken
    in bf16 (the reference's callers cast them to the autocast dtype first, block_sparse.py:947-955), products are
    accumulated in fp32.  Registered as a torch custom op with a fake implementation and the reference's backward
    (custom_ops.py:59-136)."""
    _check_meta(offsets, row_indices, column_indices)
    assert lhs.shape[1] == shape0, "incompatible dimensions"
    d = data.detach()
    if d.dim() != 3 or d.shape[1] != 16 or d.shape[2] != 16:
        raise ValueError(f"stk_dds: data must be [nnz, 16, 16] (carve(blocking=16)), got {tuple(data.shape)}")
    db = (d if d.dtype == torch.bfloat16 else d.to(torch.bfloat16)).contiguous()
    x = lhs if lhs.dtype == torch.bfloat16 else lhs.to(torch.bfloat16)
    if transpose_b:
        T = _bcsr(offsets, column_indices, int(d.shape[0]), shape1, shape0, d.device)
    else:
        T, src = _bcsr(offsets, column_indices, int(d.shape[0]), shape0, shape1, d.device).transposed()
        db = db[src].transpose(1, 2).contiguous()
    y = ops.dds_values(x, db, T)
    return y if y.dtype == lhs.dtype else y.to(lhs.dtype)


@stk_dds.register_fake
def _stk_dds_fake(lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
                  shape0, shape1, transpose_b):
    return lhs.new_empty((lhs.size(0), shape1))


def stk_dds_ternary(lhs: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor, column_indices: Tensor,
                    offsets_t: Tensor, column_indices_t: Tensor, block_offsets_t: Tensor,
                    shape0: int, shape1: int, transpose_b: bool) -> Tensor:
    """stk_dds for data that is ternary per block (every value of block j is 0 or +-s_j): same signature and result, run by
    the ternary kernels (the values are encoded on the device at every call).  Data that is not ternary is never multiplied
    approximately: the result of such a call is all NaN and a ValueError follows (see ``_pack_from_data``).  Not a torch
    custom op: no autograd; the modules' own autograd functions cover training."""
    _check_meta(offsets, row_indices, column_indices)
    assert lhs.shape[1] == shape0, "incompatible dimensions"
    if transpose_b:
        W = _pack_from_data(data, offsets, column_indices, shape1, shape0)
    else:
        W = _pack_from_data(data, offsets, column_indices, shape0, shape1, transposed=True)
    x = lhs if lhs.dtype == torch.bfloat16 else lhs.to(torch.bfloat16)
    y = ops.spmm(x, W)
    W.poison_on_status(y)
    return y if y.dtype == lhs.dtype else y.to(lhs.dtype)


@torch.library.custom_op("mortar_amd::sdd_at_b", mutates_args=(), device_types="cuda")
def stk_sdd_at_b(a: Tensor, b: Tensor, data: Tensor, offsets: Tensor, row_indices: Tensor,
                 column_indices: Tensor) -> Tensor:
    """a^T @ b restricted to the topology of ``data`` ([nnz, 16, 16], values never read): the dW product
    (reference: custom_ops.py:78-96).  a [M, rows*16], b [M, cols*16]; result in a.dtype."""
    _check_meta(offsets, row_indices, column_indices)
    if data.dim() != 3 or data.shape[1] != 16 or data.shape[2] != 16:
        raise ValueError(f"stk_sdd_at_b: data must be [nnz, 16, 16], got {tuple(data.shape)}")
    W = _topology(offsets, column_indices, int(data.shape[0]), a.shape[1], b.shape[1], a.device)
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
