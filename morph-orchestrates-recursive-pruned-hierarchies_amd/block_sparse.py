"""CMSBlockLinear: the carved (MORTAR) linear layer, runtime side.

Mirrors the carve / carved-forward / checkpoint surface of the reference's
morph/model/layers/block_sparse.py (class and buffer names are kept because other code finds the layer by
``type(m).__name__ == "CMSBlockLinear"`` and by its ``mortar_*`` attributes).  The training-time scoring and
pruning machinery of the reference class is not part of this runtime.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from .deploy_quant import _ternary_quantize, pack_ternary_codes
from .pack import MortarPack


def _stk_transpose(size, data, row_indices, column_indices, offsets):
    """Transposed-topology metadata (reference: morph/sparse/stk/matrix.py:107-125).  A stable sort fixes the
    order of blocks inside one block-column, which the reference leaves to the sort backend."""
    block_columns = size[1] // data.shape[1]
    gather_indices = torch.sort(column_indices.to(torch.int32), stable=True).indices
    column_indices_t = row_indices.gather(0, gather_indices)
    block_offsets_t = gather_indices.int()
    nnz_per_column = torch.bincount(column_indices.to(torch.int64), minlength=block_columns).int()
    zero = torch.zeros((1,), dtype=torch.int32, device=data.device)
    offsets_t = torch.cat([zero, nnz_per_column.cumsum(0, dtype=torch.int32)])
    return column_indices_t, offsets_t, block_offsets_t


class _MortarLinearFn(torch.autograd.Function):
    """y = x W^T on the carved topology with the reference's backward (morph/sparse/stk/backend/custom_ops.py:99-136):
    dx = dy W through the W^T pack, d(mortar_data) = dy^T x restricted to the kept blocks."""

    @staticmethod
    def forward(ctx, x: Tensor, data: Tensor, layer: "CMSBlockLinear") -> Tensor:
        W = layer.mortar_pack()
        ctx.layer = layer
        ctx.save_for_backward(x)
        ctx.data_dtype = data.dtype
        return ops.gemv(x, W) if 0 < x.shape[0] <= 64 else ops.spmm(x, W)

    @staticmethod
    def backward(ctx, dy: Tensor):
        (x,) = ctx.saved_tensors
        layer = ctx.layer
        dy = dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)
        dy = dy.contiguous()
        dx = ddata = None
        if ctx.needs_input_grad[0]:
            dx = ops.spmm(dy, layer.mortar_pack_t())
        if ctx.needs_input_grad[1]:
            ddata = ops.sdd(dy, x, layer.mortar_pack()).to(ctx.data_dtype)
        return dx, ddata, None


class CMSBlockLinear(nn.Module):
    def __init__(self, in_features: int, out_features: int, tile_size: int = 16, density: float = 1.0,
                 bias: bool = True, score_ema_alpha: float = 0.95, device=None, dtype=None) -> None:
        super().__init__()
        if in_features % tile_size or out_features % tile_size:
            raise ValueError(f"[{out_features},{in_features}] not divisible by tile_size {tile_size}")
        self.in_features, self.out_features, self.tile_size = in_features, out_features, tile_size
        self.R, self.C = out_features // tile_size, in_features // tile_size
        self.density = float(density)
        self.K = self.C
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=dtype))
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        self.bias = nn.Parameter(torch.zeros(out_features, device=device, dtype=dtype)) if bias else None
        self._prune_mask: Tensor | None = None       # [R, C] bool tile mask
        self._dense_mode, self._mortar, self._mortar_blocking = True, False, 0
        self._values_ternary_mode, self._values_threshold = False, 0.5
        self._pack: MortarPack | None = None
        self._pack_key = None
        self._pack_gen, self._pack_t_gen = 0, -1

    # ------------------------------------------------------------------ masks / carve

    def set_block_mask(self, block_mask: Tensor, blocking: int = 16) -> None:
        """Install a block-aligned prune mask ([out/blocking, in/blocking] bool) as the [R, C] tile mask."""
        tpb = blocking // self.tile_size
        if blocking % self.tile_size:
            raise ValueError(f"blocking ({blocking}) not divisible by tile_size ({self.tile_size})")
        self._prune_mask = block_mask.bool().repeat_interleave(tpb, 0).repeat_interleave(tpb, 1)

    def enable_values_ternary(self, threshold: float = 0.5) -> None:
        self._values_ternary_mode, self._values_threshold = True, float(threshold)
        if self._mortar:
            self.mortar_ternary.copy_(torch.tensor([1.0, threshold]))
        self._pack = None

    def carve(self, blocking: int = 16) -> int:
        """Dense masked weight -> BCSR storage in the reference's layout (block_sparse.py:810-907):
        row-major nonzero() order, int16 row/column indices, int32 offsets, data[j, lr, c] =
        W[row_j*blk+lr, col_j*blk+c], plus the transposed-topology metadata."""
        assert self._dense_mode, "carve() requires dense mode (pre-carve)"
        assert not self._mortar, "carve() already applied"
        if self.out_features % blocking or self.in_features % blocking:
            raise ValueError(f"carve: [{self.out_features},{self.in_features}] not divisible by blocking {blocking}")
        B = self.tile_size
        if blocking % B != 0:
            raise ValueError(f"carve: blocking ({blocking}) not divisible by tile_size ({B})")
        nR, nC = self.out_features // blocking, self.in_features // blocking
        with torch.no_grad():
            dense = self.weight.data
            dev = dense.device
            if self._prune_mask is None:
                kept = torch.ones(nR, nC, dtype=torch.bool, device=dev)
            else:
                tiles = self._prune_mask.to(dev)
                dense = dense * tiles.repeat_interleave(B, 0).repeat_interleave(B, 1).to(dense.dtype)
                # a carve block survives when any of the (blocking / tile_size)^2 mask tiles inside it does
                side = blocking // B
                kept = tiles.unfold(0, side, side).unfold(1, side, side).reshape(nR, nC, -1).any(dim=-1)
            per_row = kept.sum(dim=1)
            if int(per_row.min()) == 0:
                raise RuntimeError("carve: a block-row has zero kept blocks")
            rows, cols = torch.where(kept)                      # row-major order, columns ascending inside a row
            offsets = torch.zeros(nR + 1, dtype=torch.int32, device=dev)
            offsets[1:] = per_row.cumsum(0)
            # [nR, nC, blocking, blocking] view of the matrix: element [r, c, i, j] = W[r*blocking + i, c*blocking + j]
            data = dense.unfold(0, blocking, blocking).unfold(1, blocking, blocking)[rows, cols].contiguous()
            row_indices, column_indices = rows.to(torch.int16), cols.to(torch.int16)
            ct, ot, bt = _stk_transpose((self.out_features, self.in_features), data, row_indices, column_indices, offsets)
            self._init_mortar_storage(data, row_indices, column_indices, offsets, ct.contiguous(), ot.contiguous(),
                                      bt.contiguous(), blocking)
        Rb, Cb = nR, nC
        nnz = int(self.mortar_data.shape[0])
        self.density = nnz / (Rb * Cb)
        return nnz

    def _init_mortar_storage(self, data, row_indices, column_indices, offsets, column_indices_t, offsets_t,
                             block_offsets_t, blocking: int) -> None:
        if "weight" in self._parameters:
            del self._parameters["weight"]
        self.mortar_data = nn.Parameter(data)
        for name, t in (("mortar_row_indices", row_indices), ("mortar_column_indices", column_indices),
                        ("mortar_offsets", offsets), ("mortar_column_indices_t", column_indices_t),
                        ("mortar_offsets_t", offsets_t), ("mortar_block_offsets_t", block_offsets_t)):
            self.register_buffer(name, t)
        self.register_buffer("mortar_ternary", torch.tensor(
            [1.0 if self._values_ternary_mode else 0.0, self._values_threshold], dtype=torch.float32, device=data.device))
        self._mortar, self._mortar_blocking, self._dense_mode = True, int(blocking), False
        self._pack = None

    # ------------------------------------------------------------------ forward

    def get_density(self) -> float:
        return self.density

    def _mortar_effective_data(self) -> Tensor:
        """Dense-valued view of the carved weight actually used in forward ([nnz, blk, blk]); the packed
        form dequantises as bf16(code) * bf16(scale) (deploy_quant.py:367-369)."""
        if "mortar_packed" in self._buffers:
            from .deploy_quant import unpack_ternary
            w = unpack_ternary(self.mortar_packed, self._packed_numel, torch.bfloat16).view(self._packed_shape)
            s = self.mortar_scale.to(torch.bfloat16)
            return w * (s.view(-1, 1, 1) if s.dim() else s)
        d = self.mortar_data
        if not self._values_ternary_mode:
            return d
        scale = d.detach().abs().mean().clamp(min=1e-8)
        d_norm = d / scale
        q = torch.sign(d_norm) * (d_norm.abs() > self._values_threshold).to(d.dtype)
        return d + (scale * q - d).detach()

    def mortar_pack(self) -> MortarPack:
        """Device weight format for the HIP kernels.  A deployed layer (mortar_packed / mortar_scale) is packed once
        on the host.  A layer in values-ternary QAT keeps its topology packed once and has the values ternarised and
        encoded on the device whenever ``mortar_data`` changed (one launch instead of the reference's per-forward
        torch ternarisation, block_sparse.py:909-919)."""
        if not self._mortar:
            raise RuntimeError("mortar_pack() requires a carved layer")
        if self._mortar_blocking != 16:
            return self._mortar_pack_recut()
        if "mortar_packed" in self._buffers:
            if self._pack is None:
                self._pack = MortarPack(self.mortar_packed, self.mortar_scale, self.mortar_column_indices, self.mortar_offsets,
                                        self.out_features, self.in_features, self.mortar_offsets.device)
            return self._pack
        if not self._values_ternary_mode:
            raise RuntimeError("carved layer holds non-ternary values: call pack_mortar_ternary() or "
                               "enable_values_ternary() first (the MORTAR runtime executes ternary blocks only)")
        d = self.mortar_data
        if not d.is_cuda:
            if self._pack is None:        # host path (no GPU): pack once from the current values
                q, scale = _ternary_quantize(d.data, self._values_threshold)
                self._pack = MortarPack(pack_ternary_codes(q), scale, self.mortar_column_indices, self.mortar_offsets,
                                        self.out_features, self.in_features, d.device)
            return self._pack
        if self._pack is None:
            self._pack = MortarPack(None, None, self.mortar_column_indices, self.mortar_offsets, self.out_features,
                                    self.in_features, d.device)
            self._pack_key = None
            self._pack_gen, self._pack_t_gen = 0, -1
        key = (d.data_ptr(), d._version)
        if self._pack_key != key:
            self._pack_scale = self._pack.requantize(self._values(), threshold=self._values_threshold, sync=False)
            self._pack_key = key
            self._pack_gen += 1
        return self._pack

    def _mortar_pack_recut(self) -> MortarPack:
        """Pack of a layer carved at a coarser blocking (the reference's checkpoints use carve(blocking=128),
        block_sparse.py:810, pruning.py:85,248): the ternary codes are formed as the reference forms them (the packed
        buffer as stored, or mortar_data through the per-tensor rule of block_sparse.py:909-919), then every block is
        re-cut into 16 x 16 blocks on the host, all-zero sub-blocks dropped.  Inference only: the pack is rebuilt when
        mortar_data changes (address, version), and the autograd path needs carve(blocking=16)."""
        B = self._mortar_blocking
        if B % 16:
            raise ValueError(f"the gfx950 MORTAR runtime runs 16 x 16 blocks; a layer carved at {B} cannot be re-cut")
        from .pack import recut_blocks
        from .deploy_quant import unpack_ternary
        if "mortar_packed" in self._buffers:
            key = ("packed",)
            if self._pack is not None and self._pack_key == key:
                return self._pack
            q = unpack_ternary(self.mortar_packed.cpu(), self._packed_numel, torch.int8).view(self._packed_shape)
            scale = self.mortar_scale.detach().float().cpu()
        else:
            if not self._values_ternary_mode:
                raise RuntimeError("carved layer holds non-ternary values: call pack_mortar_ternary() or "
                                   "enable_values_ternary() first (the MORTAR runtime executes ternary blocks only)")
            d = self.mortar_data
            key = (d.data_ptr(), d._version)
            if self._pack is not None and self._pack_key == key:
                return self._pack
            q, scale = _ternary_quantize(d.data, self._values_threshold)
            q, scale = q.cpu(), scale.cpu()
        c16, s16, col16, off16 = recut_blocks(q.numpy(), scale.numpy(), self.mortar_row_indices.cpu().numpy(),
                                              self.mortar_column_indices.cpu().numpy(), self.out_features)
        self._pack = MortarPack(pack_ternary_codes(torch.from_numpy(c16)), torch.from_numpy(np.asarray(s16, np.float32)),
                                col16, off16, self.out_features, self.in_features, self.mortar_offsets.device,
                                allow_empty_rows=True)
        self._pack_key = key
        return self._pack

    def invalidate_pack(self) -> None:
        """Forces the next mortar_pack() of a QAT layer to re-encode the values.  Writes through ``mortar_data.data``
        (EMA swaps, manual re-initialisation, ``p.data.mul_``) do not advance the parameter's version counter, so the
        (address, version) key alone would miss them; every training forward therefore calls this first (the re-encode
        is two small launches and no synchronisation)."""
        self._pack_key = None

    def mortar_pack_t(self) -> MortarPack:
        """The pack of W^T for the dX product (QAT layers on the GPU), refreshed like ``mortar_pack``."""
        if "mortar_packed" in self._buffers or not self.mortar_data.is_cuda:
            raise RuntimeError("mortar_pack_t(): the backward needs a QAT layer (mortar_data) on the GPU")
        t = self.mortar_pack().transposed()
        if self._pack_t_gen != self._pack_gen:
            t.requantize(self._values(), threshold=self._values_threshold, scale=self._pack_scale, transpose=True,
                         sync=False)              # the scale W was packed with: no second reduction over the values
            self._pack_t_gen = self._pack_gen
        return t

    def _values(self) -> Tensor:
        d = self.mortar_data.detach()
        if d.dtype not in (torch.bfloat16, torch.float32):
            d = d.float()
        return d.contiguous()

    def _forward_mortar(self, x: Tensor) -> Tensor:
        """Carved forward y = x @ W_sparse^T (+bias).  Reference: block_sparse.py:921-970 (flatten leading
        dims, bf16 operands, fp32 accumulate, output in the activation dtype; no M padding is needed).  With autograd
        on a QAT layer the backward runs dX through the W^T pack and dW through the topology-restricted product
        (reference: custom_ops.py:99-136), the gradient passing straight through the ternarisation into mortar_data."""
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        xb = x2 if x2.dtype == torch.bfloat16 else x2.to(torch.bfloat16)
        trainable = ("mortar_packed" not in self._buffers and self._values_ternary_mode and xb.is_cuda
                     and self._mortar_blocking == 16)
        if (not trainable and self._mortar_blocking != 16 and torch.is_grad_enabled()
                and (xb.requires_grad or ("mortar_data" in self._parameters and self.mortar_data.requires_grad))):
            raise RuntimeError(f"autograd through a layer carved at blocking {self._mortar_blocking}: the backward runs on "
                               "carve(blocking=16) layers only (re-cut packs serve inference)")
        if trainable and self.mortar_data.requires_grad:
            self.invalidate_pack()            # trainable values may have been written through .data since the last call
        if trainable and torch.is_grad_enabled() and (xb.requires_grad or self.mortar_data.requires_grad):
            y = _MortarLinearFn.apply(xb, self.mortar_data, self)
        else:
            W = self.mortar_pack()
            y = ops.gemv(xb, W) if 0 < xb.shape[0] <= 64 else ops.spmm(xb, W)
        if y.dtype != x.dtype:
            y = y.to(x.dtype)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)

    def forward(self, x: Tensor) -> Tensor:
        if self._mortar:
            return self._forward_mortar(x)
        w = self.weight
        if self._prune_mask is not None:
            B = self.tile_size
            w = w * self._prune_mask.to(w.device).repeat_interleave(B, 0).repeat_interleave(B, 1).to(w.dtype)
        return F.linear(x, w, self.bias)

    def _apply(self, fn, *a, **k):
        self._pack = None       # device may change
        return super()._apply(fn, *a, **k)

    # ------------------------------------------------------------------ checkpoints

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        """Accepts the reference's carved key set (block_sparse.py:983-1036): mortar_data + six index buffers
        + mortar_ternary, or the packed variant mortar_packed + mortar_scale in place of mortar_data."""
        dk, pk = prefix + "mortar_data", prefix + "mortar_packed"
        if (dk in state_dict or pk in state_dict) and not self._mortar:
            dev = self.weight.device
            idx = {k: torch.empty_like(state_dict[prefix + k], device=dev) for k in (
                "mortar_row_indices", "mortar_column_indices", "mortar_offsets", "mortar_column_indices_t",
                "mortar_offsets_t", "mortar_block_offsets_t")}
            mt = state_dict.get(prefix + "mortar_ternary")
            if mt is not None:
                self._values_ternary_mode = bool(float(mt[0]) > 0)
                self._values_threshold = float(mt[1])
            nnz = int(idx["mortar_row_indices"].numel())
            if dk in state_dict:
                ck = state_dict[dk]
                blocking = int(ck.shape[-1])
                data = torch.empty_like(ck, device=dev)
            else:
                blocking = int(round(math.sqrt(state_dict[pk].numel() * 4 / max(nnz, 1))))
                data = torch.empty(0, device=dev)
            self._init_mortar_storage(data, idx["mortar_row_indices"], idx["mortar_column_indices"],
                                      idx["mortar_offsets"], idx["mortar_column_indices_t"], idx["mortar_offsets_t"],
                                      idx["mortar_block_offsets_t"], blocking)
            if pk in state_dict and dk not in state_dict:
                del self._parameters["mortar_data"]
                self.register_buffer("mortar_packed", torch.empty_like(state_dict[pk], device=dev))
                self.register_buffer("mortar_scale", torch.empty_like(state_dict[prefix + "mortar_scale"], device=dev))
                self._packed_shape = (nnz, blocking, blocking)
                self._packed_numel = nnz * blocking * blocking
            Rb, Cb = self.out_features // blocking, self.in_features // blocking
            self.density = nnz / (Rb * Cb)
        self._pack = None
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, tile_size={self.tile_size}, "
                f"density={self.density:.2f}, mortar={self._mortar}, bias={self.bias is not None}")
