"""Device-side weight format of one carved matrix, built once from the reference's carve output.

Counterpart of the reference's one-time engine re-pack (mortar_pack_strips,
morph/kernels/triton/fused_decode_step.py:1465-1499): the ternary codes keep their BCSR order, the
reference's ``mortar_column_indices`` (int16) and ``mortar_offsets`` (int32) are uploaded unchanged, and
only the bit layout inside each block-row dword and the scale pattern are device specific.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib

BLK = 16
SCHED_GROUP = 16      # wavefronts of a prefill workgroup: the group size of the row-unit order
SCHED_UNITS_PER_WAVE = {1: 4, 2: 2}   # units a wave of the K-segmented prefill kernel owns, by rows per unit


def _np(a, dtype):
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return np.ascontiguousarray(a, dtype=dtype)


def _vp(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def encode_blocks(packed, nnz: int, scale) -> tuple[np.ndarray, np.ndarray]:
    """Reference flat 2-bit pack + scale(s) -> (device code dwords [nnz*16] uint32, scale patterns [nnz] uint32)."""
    packed = _np(packed, np.uint8).reshape(-1)
    if packed.size < nnz * 64:
        raise ValueError(f"packed codes hold {packed.size} bytes, need {nnz * 64}")
    scale = _np(scale, np.float32).reshape(-1)
    codes = np.empty(nnz * 16, dtype=np.uint32)
    sdup = np.empty(nnz, dtype=np.uint32)
    _lib.check(_lib.lib().mortar_encode_blocks_host(_vp(packed), nnz, _vp(scale), scale.size, _vp(codes), _vp(sdup)),
               "mortar_encode_blocks_host")
    return codes, sdup


def decode_blocks(codes: np.ndarray) -> np.ndarray:
    codes = _np(codes, np.uint32).reshape(-1)
    nnz = codes.size // 16
    out = np.empty((nnz, 16, 16), dtype=np.int8)
    _lib.check(_lib.lib().mortar_decode_blocks_host(_vp(codes), nnz, _vp(out)), "mortar_decode_blocks_host")
    return out


def validate_bcsr(offsets, col, Rb: int, Cb: int) -> None:
    offsets, col = _np(offsets, np.int32), _np(col, np.int16)
    _lib.check(_lib.lib().mortar_validate_bcsr_host(_vp(offsets), _vp(col), Rb, Cb), "mortar_validate_bcsr_host")


def octet_layout(offsets, Rb: int, Cb: int, seg_cb: int, codes: np.ndarray, sdup: np.ndarray, col):
    """-> (row_desc [nseg*Rb*4] int32, codes_o uint32, sd_o uint32, col_o int32): see mortar_octet_layout_host."""
    offsets, col = _np(offsets, np.int32), _np(col, np.int16)
    codes, sdup = _np(codes, np.uint32), _np(sdup, np.uint32)
    L = _lib.lib()
    nseg = -(-Cb // seg_cb)
    grp = np.empty(nseg * Rb * 4, dtype=np.int32)
    ng = _lib.check(L.mortar_octet_layout_host(_vp(offsets), Rb, Cb, seg_cb, None, None, _vp(col), _vp(grp), None, None, None),
                    "mortar_octet_layout_host")
    codes_o = np.empty(ng * 128, dtype=np.uint32)
    sd_o = np.empty(ng * 8, dtype=np.uint32)
    col_o = np.empty(ng * 8, dtype=np.int32)
    _lib.check(L.mortar_octet_layout_host(_vp(offsets), Rb, Cb, seg_cb, _vp(codes), _vp(sdup), _vp(col), _vp(grp),
                                          _vp(codes_o), _vp(sd_o), _vp(col_o)), "mortar_octet_layout_host")
    return grp, codes_o, sd_o, col_o


def fp4_stream(codes_o: np.ndarray) -> np.ndarray:
    """4-bit (FP4) copy of an octet code stream: see mortar_fp4_stream_host."""
    codes_o = _np(codes_o, np.uint32)
    out = np.empty(codes_o.size * 2, dtype=np.uint32)
    _lib.check(_lib.lib().mortar_fp4_stream_host(_vp(codes_o), codes_o.size // 128, _vp(out)), "mortar_fp4_stream_host")
    return out


def octet_positions(offsets, Rb: int, Cb: int, seg_cb: int, col) -> np.ndarray:
    """Index of every block in the octet streams: see mortar_octet_positions_host."""
    offsets, col = _np(offsets, np.int32), _np(col, np.int16)
    out = np.empty(col.size, dtype=np.int32)
    _lib.check(_lib.lib().mortar_octet_positions_host(_vp(offsets), Rb, Cb, seg_cb, _vp(col), _vp(out)),
               "mortar_octet_positions_host")
    return out


def transpose_topology(offsets, col, Rb: int, Cb: int):
    """-> (offsets_t [Cb+1] int32, col_t [nnz] int16, src_block [nnz] int32): see mortar_transpose_topology_host."""
    offsets, col = _np(offsets, np.int32), _np(col, np.int16)
    off_t = np.empty(Cb + 1, dtype=np.int32)
    col_t = np.empty(col.size, dtype=np.int16)
    src = np.empty(col.size, dtype=np.int32)
    _lib.check(_lib.lib().mortar_transpose_topology_host(_vp(offsets), _vp(col), Rb, Cb, _vp(off_t), _vp(col_t), _vp(src)),
               "mortar_transpose_topology_host")
    return off_t, col_t, src


def recut_blocks(codes: np.ndarray, scales, row_idx, col_idx, out_features: int, blk: int = BLK):
    """A BCSR carved at a coarser blocking B (the reference's default is carve(blocking=128), block_sparse.py:810,
    pruning.py:85) re-cut into the 16 x 16 blocks the kernels run: block j at (R, C) becomes its (B/16)^2 sub-blocks at
    (R*B/16 + sr, C*B/16 + sc); sub-blocks whose codes are all zero are dropped, so that pruned 16 x 16 tiles inside a
    kept coarse block cost nothing.  codes int8 [nnz, B, B]; scales scalar or [nnz] (a sub-block inherits its block's).
    Returns (codes16 int8 [nnz16, 16, 16], scales16 fp32 scalar or [nnz16], col16 int16 [nnz16], offsets16 int32
    [out_features/16 + 1]) in row-major order, columns ascending inside a row.  Rows of 16 may end up empty."""
    codes = np.asarray(codes)
    nnz, B, _ = codes.shape
    if B % blk or codes.shape[2] != B:
        raise ValueError(f"recut_blocks: blocks of {codes.shape[1:]} are not multiples of {blk}")
    s = B // blk
    sub = codes.reshape(nnz, s, blk, s, blk).transpose(0, 1, 3, 2, 4)                 # [nnz, sr, sc, 16, 16]
    keep = sub.reshape(nnz, s, s, -1).any(axis=-1)
    r16 = (np.asarray(row_idx, np.int64)[:, None, None] * s + np.arange(s)[None, :, None]) + np.zeros((1, 1, s), np.int64)
    c16 = (np.asarray(col_idx, np.int64)[:, None, None] * s + np.arange(s)[None, None, :]) + np.zeros((1, s, 1), np.int64)
    j, sr, sc = np.nonzero(keep)
    rr, cc = r16[j, sr, sc], c16[j, sr, sc]
    order = np.lexsort((cc, rr))
    Rb16 = out_features // blk
    offsets = np.zeros(Rb16 + 1, np.int32)
    offsets[1:] = np.cumsum(np.bincount(rr, minlength=Rb16))
    sc_arr = np.asarray(scales, np.float32).reshape(-1)
    scales16 = sc_arr if sc_arr.size == 1 else sc_arr[j[order]]
    return (np.ascontiguousarray(sub[j, sr, sc][order]), scales16, cc[order].astype(np.int16), offsets)


def unit_order(offsets, Rb: int, rows_per_unit: int, group: int = SCHED_GROUP, snake: bool = True) -> np.ndarray:
    """Row units by schedule position (mortar_unit_order_host): ``snake`` reverses the odd groups, for the kernels
    that give wave w the positions w, w + group, ... of a window (matrices with several K segments)."""
    offsets = _np(offsets, np.int32)
    out = np.empty(Rb // rows_per_unit, dtype=np.int32)
    _lib.check(_lib.lib().mortar_unit_order_host(_vp(offsets), Rb, rows_per_unit, group, 1 if snake else 0, _vp(out)),
               "mortar_unit_order_host")
    return out


def unit_order_segments(row_desc, Rb: int, nseg: int, rows_per_unit: int, order: np.ndarray) -> np.ndarray:
    """Re-deal every workgroup window of ``order`` so that no wave is the slowest in every K segment."""
    row_desc, out = _np(row_desc, np.int32), _np(order, np.int32).copy()
    _lib.check(_lib.lib().mortar_unit_order_segments_host(_vp(row_desc), Rb, nseg, rows_per_unit, SCHED_GROUP,
                                                          SCHED_UNITS_PER_WAVE[rows_per_unit], _vp(out)),
               "mortar_unit_order_segments_host")
    return out


def schedule(row_desc: np.ndarray, Rb: int, nseg: int, rows_per_unit: int, order: np.ndarray | None) -> np.ndarray:
    """Part descriptors in schedule order [n_units, nseg, rows_per_unit, 4] int32: see mortar_schedule_host."""
    row_desc = _np(row_desc, np.int32)
    out = np.empty((Rb // rows_per_unit, nseg, rows_per_unit, 4), dtype=np.int32)
    o = _np(order, np.int32) if order is not None else None
    _lib.check(_lib.lib().mortar_schedule_host(_vp(row_desc), Rb, nseg, rows_per_unit, _vp(o) if o is not None else None,
                                               _vp(out)), "mortar_schedule_host")
    return out


def decode_worklist(offsets, col, Rb: int, Cb: int, rows_per_unit: int, kseg: int, max_blocks: int):
    """-> (entries [E, 8] int32, nslots, row_slots [Rb] int32).  See mortar_decode_worklist_host."""
    offsets, col = _np(offsets, np.int32), _np(col, np.int16)
    L = _lib.lib()
    ns = C.c_int32(0)
    n = _lib.check(L.mortar_decode_worklist_host(_vp(offsets), _vp(col), Rb, Cb, rows_per_unit, kseg, max_blocks,
                                                 None, C.byref(ns), None), "mortar_decode_worklist_host")
    ent = np.empty((n, 8), dtype=np.int32)
    row_slots = np.empty(Rb, dtype=np.int32)
    _lib.check(L.mortar_decode_worklist_host(_vp(offsets), _vp(col), Rb, Cb, rows_per_unit, kseg, max_blocks,
                                             _vp(ent), C.byref(ns), _vp(row_slots)), "mortar_decode_worklist_host")
    return ent, int(ns.value), row_slots


class BcsrTopology:
    """The reference's BCSR index arrays of one matrix (mortar_offsets, mortar_column_indices) on the device, with what the
    product over stored block values needs beside them: the per-segment row pointers for wide K and the transposed topology
    (reference: stk matrix.py:107-125) for the dX product.  No codes, no scales: the values stay where the caller has them."""

    def __init__(self, offsets, col, out_features: int, in_features: int, device):
        if out_features % BLK or in_features % BLK:
            raise ValueError(f"[{out_features},{in_features}] not divisible by blocking {BLK}")
        self.out_features, self.in_features = int(out_features), int(in_features)
        self.Rb, self.Cb = out_features // BLK, in_features // BLK
        self.h_offsets = _np(offsets, np.int32).reshape(-1)
        self.h_col = _np(col, np.int16).reshape(-1)
        if self.h_offsets.size != self.Rb + 1:
            raise ValueError(f"offsets has {self.h_offsets.size} entries, expected {self.Rb + 1}")
        self.nnz = int(self.h_offsets[-1])
        if self.h_col.size != self.nnz:
            raise ValueError(f"column_indices has {self.h_col.size} entries, offsets say {self.nnz}")
        validate_bcsr(self.h_offsets, self.h_col, self.Rb, self.Cb)
        self.device = torch.device(device)
        self.row_ptr = torch.from_numpy(self.h_offsets).to(self.device)
        self.col = torch.from_numpy(self.h_col).to(self.device)
        L = _lib.lib()
        self.seg_cb = int(L.mortar_values_seg_cb(self.Cb))
        self.nseg = -(-self.Cb // self.seg_cb)
        self.seg_ptr = None
        if self.nseg > 1:
            sp = np.empty(self.Rb * (self.nseg + 1), dtype=np.int32)
            _lib.check(L.mortar_segment_ptr_host(_vp(self.h_offsets), _vp(self.h_col), self.Rb, self.Cb, self.seg_cb, _vp(sp)),
                       "mortar_segment_ptr_host")
            self.seg_ptr = torch.from_numpy(sp).to(self.device)
        self._t = None

    def transposed(self):
        """(topology of W^T, src): block j of W^T is block src[j] of W, transposed (int64 device index)."""
        if self._t is None:
            off_t, col_t, src = transpose_topology(self.h_offsets, self.h_col, self.Rb, self.Cb)
            self._t = (BcsrTopology(off_t, col_t, self.in_features, self.out_features, self.device),
                       torch.from_numpy(src.astype(np.int64)).to(self.device))
        return self._t


class MortarPack:
    """One carved matrix W [out, in] resident on a device, plus its cached schedules.

    Built from the reference's buffers: ``packed`` = mortar_packed (flat 2-bit codes over [nnz,16,16]),
    ``scale`` = mortar_scale (scalar) or a per-block fp32 vector, ``col`` = mortar_column_indices,
    ``offsets`` = mortar_offsets.  ``prefill_stream`` also keeps the 4-bit copy of the code stream that
    prefill-sized launches (M > 64) unpack faster (+128 bytes per block of device memory); without it they
    unpack the 2-bit stream.  When all blocks share one scale (the reference's per-tensor mortar_scale) and
    ``scale_after_sum`` is on, the kernels scale the fp32 sums once instead of every block's weights
    (``uniform_scale``; about a third fewer vector instructions per block pair).

    ``seg_cb`` sets the width of the stream's K segments in block-columns (default: the widest whose 32-token
    activation tile fits LDS, ``mortar_prefill_max_seg_cb()``).

    ``packed=None`` builds the topology with all-zero blocks, to be filled on the device by ``requantize`` from
    block values (the reference's ``mortar_data``): the device-side pack used for QAT forwards and for the W^T
    pack of the dX product (``transposed()``).
    """

    def __init__(self, packed, scale, col, offsets, out_features: int, in_features: int, device,
                 prefill_stream: bool = True, scale_after_sum: bool = True, allow_empty_rows: bool = False,
                 seg_cb: int | None = None, decode_rows: int = 0):
        if out_features % BLK or in_features % BLK:
            raise ValueError(f"[{out_features},{in_features}] not divisible by blocking {BLK}")
        self.out_features, self.in_features = int(out_features), int(in_features)
        self.Rb, self.Cb = out_features // BLK, in_features // BLK
        self.h_offsets = _np(offsets, np.int32).reshape(-1)
        self.h_col = _np(col, np.int16).reshape(-1)
        if self.h_offsets.size != self.Rb + 1:
            raise ValueError(f"offsets has {self.h_offsets.size} entries, expected {self.Rb + 1}")
        self.nnz = int(self.h_offsets[-1])
        if self.h_col.size != self.nnz:
            raise ValueError(f"column_indices has {self.h_col.size} entries, offsets say {self.nnz}")
        if (np.diff(self.h_offsets) <= 0).any() and not allow_empty_rows:       # the reference's carve refuses these
            raise RuntimeError("carved matrix has a block-row with zero kept blocks")
        self.device = torch.device(device)
        if packed is None:
            codes, sdup = np.zeros(self.nnz * 16, dtype=np.uint32), np.zeros(self.nnz, dtype=np.uint32)
            self.scales_f32 = None
        else:
            codes, sdup = encode_blocks(packed, self.nnz, scale)
            # the scales as given (fp32, not rounded to bf16): what the fp32 decode arithmetic multiplies by
            sc = scale.detach().cpu().numpy() if isinstance(scale, torch.Tensor) else np.asarray(scale)
            self.scales_f32 = torch.from_numpy(np.ascontiguousarray(sc, dtype=np.float32).reshape(-1)).to(self.device)
        validate_bcsr(self.h_offsets, self.h_col, self.Rb, self.Cb)
        us = C.c_float(0.0)
        _lib.check(_lib.lib().mortar_uniform_scale_host(_vp(sdup), self.nnz, C.byref(us)), "mortar_uniform_scale_host")
        self.scale_after_sum = bool(scale_after_sum)
        self.uniform_scale = float(us.value) if scale_after_sum else 0.0
        dev = self.device
        self.codes = torch.from_numpy(codes.view(np.int32)).to(dev)
        self.sdup = torch.from_numpy(sdup.view(np.int32)).to(dev)
        self.col = torch.from_numpy(self.h_col).to(dev)
        self.row_ptr = torch.from_numpy(self.h_offsets).to(dev)
        max_seg = int(_lib.lib().mortar_decode_max_seg_cb(decode_rows) if decode_rows else _lib.lib().mortar_prefill_max_seg_cb())
        self.decode_rows = int(decode_rows)     # > 0: K segments wider than a 32-token tile allows; calls of up to that many rows
        if seg_cb is not None:
            if not 0 < seg_cb <= max_seg:
                raise ValueError(f"seg_cb={seg_cb} outside 1..{max_seg}")
            nseg = -(-self.Cb // seg_cb)
            self.seg_cb = int(seg_cb)
        else:
            nseg = -(-self.Cb // max_seg)
            self.seg_cb = -(-self.Cb // nseg)
        grp, codes_o, sd_o, col_o = octet_layout(self.h_offsets, self.Rb, self.Cb, self.seg_cb, codes, sdup, self.h_col)
        self.nseg = nseg
        self.h_row_desc = grp
        self.row_desc = torch.from_numpy(grp).to(dev)
        self.codes_o = torch.from_numpy(codes_o.view(np.int32)).to(dev)
        self.sd_o = torch.from_numpy(sd_o.view(np.int32)).to(dev)
        self.col_o = torch.from_numpy(col_o).to(dev)
        self.codes4_o = torch.from_numpy(fp4_stream(codes_o).view(np.int32)).to(dev) if prefill_stream else None
        self._scheds: dict[int, torch.Tensor] = {}
        self._worklists: dict[tuple, tuple] = {}
        # what decode_view() rebuilds the stream from; dropped once the values are rewritten on the device
        self._h_codes, self._h_sdup, self._dview = (codes, sdup, {}) if packed is not None else (None, None, {})
        self._pos = self._ws = self._status = self.src_block = self._sdd = None
        self._status_host = self._status_event = None
        self._transposed: "MortarPack | None" = None
        self.struct = self._make_struct()
        self.ref = C.byref(self.struct)

    def _make_struct(self):
        return _lib.BcsrStruct(self.codes.data_ptr(), self.sdup.data_ptr(), self.col.data_ptr(),
                               self.row_ptr.data_ptr(), self.row_desc.data_ptr(), self.codes_o.data_ptr(),
                               self.sd_o.data_ptr(), self.col_o.data_ptr(),
                               self.codes4_o.data_ptr() if self.codes4_o is not None else None,
                               self.Rb, self.Cb, self.nnz, self.seg_cb, self.uniform_scale, 0)

    def decode_view(self, rows: int) -> "MortarPack | None":
        """A second stream of this matrix for calls of up to 4 rows: K segments as wide as a 4-token tile allows (one
        segment for rows of up to 19840 values), so a row is one part and is padded to octets once.  Shares the topology and
        code arrays; costs 72 bytes per block.  None for more rows (a two-segment stream for 16-token tiles was measured
        slower than the three-segment one: its 90 KB tile leaves one workgroup per CU), when it would not reduce the number
        of segments, or when the values were rewritten on the device (the view is built from the host copy of the codes)."""
        if rows > 4 or self.decode_rows or self._h_codes is None:
            return None
        tile = 4
        nseg = -(-self.Cb // int(_lib.lib().mortar_decode_max_seg_cb(tile)))
        if nseg >= self.nseg:
            return None
        if tile not in self._dview:
            v = object.__new__(MortarPack)
            v.__dict__.update(self.__dict__)
            v.decode_rows, v.seg_cb, v.nseg = tile, -(-self.Cb // nseg), nseg
            grp, codes_o, sd_o, col_o = octet_layout(self.h_offsets, self.Rb, self.Cb, v.seg_cb, self._h_codes, self._h_sdup, self.h_col)
            v.h_row_desc = grp
            v.row_desc = torch.from_numpy(grp).to(self.device)
            v.codes_o = torch.from_numpy(codes_o.view(np.int32)).to(self.device)
            v.sd_o = torch.from_numpy(sd_o.view(np.int32)).to(self.device)
            v.col_o = torch.from_numpy(col_o).to(self.device)
            v.codes4_o = None
            v._scheds, v._worklists, v._transposed, v._dview = {}, {}, None, {}
            v._h_codes = v._h_sdup = None
            v.struct = v._make_struct()
            v.ref = C.byref(v.struct)
            self._dview[tile] = v
        return self._dview[tile]

    # ---- device-side re-pack ----------------------------------------------------------------------------------

    def requantize(self, values: torch.Tensor, per_block: bool = False, threshold: float = 0.5,
                   scale: torch.Tensor | None = None, transpose: bool = False, sync: bool = True,
                   ternary_tol: float = 0.0) -> torch.Tensor:
        """Ternarise ``values`` [nnz,16,16] (bf16 or fp32, on this device) into this pack, in place, on the current
        stream: scale = mean|w| over the matrix (reference deploy_quant.py:81-95, block_sparse.py:909-919) or per
        block (``per_block``), or the given ``scale`` (fp32 [1] or [nnz], indexed like ``values``); code =
        sign(w/s) * (|w/s| > threshold).  A pack from ``transposed()`` reads the blocks of the original matrix
        (its ``src_block`` map) and pass ``transpose=True``.  Returns the scale tensor (fp32 [1] or [nnz], in this
        pack's block order).  ``sync=True`` waits, raises if a scale left the representable window, and selects the
        scale-after-sum kernels for a one-scale matrix; ``sync=False`` only enqueues (per-block kernels) and lets the
        device status word accumulate: ``poll_status()`` / ``raise_status()`` report it later.
        ``ternary_tol`` > 0 (with a given ``scale``): values that are neither 0 nor +-scale within that relative bound
        are reported as an error (the values are expected to be ternary already)."""
        if values.device != self.device or values.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("requantize: values must be bf16 or fp32 on the pack's device")
        if tuple(values.shape) != (self.nnz, BLK, BLK) or not values.is_contiguous():
            raise ValueError(f"requantize: values must be contiguous [{self.nnz}, 16, 16], got {tuple(values.shape)}")
        self._h_codes, self._h_sdup, self._dview = None, None, {}      # the host copy of the codes is stale from here on
        L = _lib.lib()
        if self._pos is None:
            self._pos = torch.from_numpy(octet_positions(self.h_offsets, self.Rb, self.Cb, self.seg_cb, self.h_col)).to(self.device)
            self._ws = torch.empty(int(L.mortar_requantize_workspace_bytes()) // 8, dtype=torch.float64, device=self.device)
            self._status = torch.zeros(2, dtype=torch.int32, device=self.device)
        if scale is not None:
            scale = scale.detach().to(device=self.device, dtype=torch.float32).reshape(-1).contiguous()
            if scale.numel() not in (1, self.nnz):
                raise ValueError(f"requantize: scale must have 1 or {self.nnz} entries")
            mode = 2 if scale.numel() == 1 else 3
        else:
            mode = 1 if per_block else 0
        if ternary_tol and scale is None:
            raise ValueError("requantize: ternary_tol needs a given scale")
        out = torch.empty(1 if mode in (0, 2) else self.nnz, dtype=torch.float32, device=self.device)
        st = torch.cuda.current_stream(self.device).cuda_stream
        if sync and self._status_host is not None:
            self.raise_status()          # a synchronous call clears the words: report what earlier asynchronous calls left first
        # asynchronous calls leave the status words sticky (flags bit 0) so that a later poll still sees a failure
        _lib.check(L.mortar_requantize(self.ref, values.data_ptr(), int(values.dtype == torch.float32), self._pos.data_ptr(),
                                       self.src_block.data_ptr() if self.src_block is not None else None,
                                       int(bool(transpose)), mode, float(threshold),
                                       scale.data_ptr() if scale is not None else None, out.data_ptr(),
                                       self._status.data_ptr(), 0 if sync else 1, float(ternary_tol),
                                       self._ws.data_ptr(), st), "mortar_requantize")
        self.scales_f32 = out
        us = 0.0
        if sync:
            self.raise_status()
            if mode in (0, 2) and self.scale_after_sum:
                us = float(out.to(torch.bfloat16).float().item())
        elif ternary_tol:
            self._post_status()
        if us != self.uniform_scale:
            self.uniform_scale = us
            self.struct.uniform_scale = us
        return out

    # status of asynchronous re-packs: the device words are copied to pinned host memory behind every call; reading them
    # costs no synchronisation once the copy has landed

    def _post_status(self) -> None:
        if torch.cuda.is_current_stream_capturing():       # a captured step keeps the words on the device only
            return
        if self._status_host is None:
            self._status_host = torch.zeros(2, dtype=torch.int32, pin_memory=True)
            self._status_event = torch.cuda.Event()
        self._status_host.copy_(self._status, non_blocking=True)
        self._status_event.record(torch.cuda.current_stream(self.device))

    @staticmethod
    def _status_error(flags) -> str | None:
        if flags[1]:
            return "values are not ternary per block (+-s_j or 0) for the given scale; quantise them first"
        if flags[0]:
            return "a block scale lies outside [2^-100, 2^100] (block zeroed)"
        return None

    def poll_status(self) -> str | None:
        """Error text of an earlier asynchronous requantize whose status has reached the host, else None.  Never waits.
        The device words are cleared once an error has been reported."""
        if self._status_host is None or not self._status_event.query():
            return None
        msg = self._status_error(self._status_host.tolist())
        if msg is not None:
            self._status.zero_()
            self._status_host.zero_()
        return msg

    def raise_status(self) -> None:
        """Waits for the re-packs enqueued so far and raises ValueError if one of them reported an error."""
        if self._status is None:
            return
        msg = self._status_error(self._status.tolist())
        if msg is not None:
            self._status.zero_()
            if self._status_host is not None:
                self._status_host.zero_()
            raise ValueError("requantize: " + msg)

    def poison_on_status(self, out: torch.Tensor) -> None:
        """Enqueues the device-side check behind a product of this pack: ``out`` becomes all NaN if a re-pack of this pack
        has reported an error that has not been raised yet (no host synchronisation).  No-op for packs never re-packed."""
        if self._status is None:
            return
        if not out.is_contiguous() or (out.numel() * out.element_size()) % 4:
            raise ValueError("poison_on_status: out must be contiguous with a multiple of 4 bytes")
        _lib.check(_lib.lib().mortar_poison_on_status(out.data_ptr(), out.numel() * out.element_size(), self._status.data_ptr(),
                                                      torch.cuda.current_stream(self.device).cuda_stream), "mortar_poison_on_status")

    def transposed(self) -> "MortarPack":
        """The pack of W^T [in, out] over the transposed topology (reference: stk matrix.py:107-125), all-zero until
        ``requantize(values_of_W, transpose=True)`` fills it.  x_grad = y_grad @ W is ``ops.spmm(y_grad, W.transposed())``:
        the reference's stk_dds(..., transpose_b=False)."""
        if self._transposed is None:
            off_t, col_t, src = transpose_topology(self.h_offsets, self.h_col, self.Rb, self.Cb)
            t = MortarPack(None, None, col_t, off_t, self.in_features, self.out_features, self.device,
                           prefill_stream=self.codes4_o is not None, scale_after_sum=self.scale_after_sum,
                           allow_empty_rows=True)        # a block-column of W without blocks: that slice of dX is 0
            t.src_block = torch.from_numpy(src).to(self.device)
            self._transposed = t
        return self._transposed

    def sdd_plan(self, M: int, blocks_per_wave: int | None = None) -> tuple[torch.Tensor, int, int]:
        """(device plan, workgroups, blocks per wavefront) of the weight-gradient kernel for this topology at M tokens:
        see mortar_sdd_blocks_per_wave_host and mortar_sdd_plan_host.  One plan per group size is kept;
        `blocks_per_wave` overrides the choice (any built size gives the same gradient)."""
        L = _lib.lib()
        if self._sdd is None:
            self._sdd = {}
        nb = blocks_per_wave if blocks_per_wave is not None else self._sdd.get(("M", M))
        if nb is None:
            nb = _lib.check(L.mortar_sdd_blocks_per_wave_host(_vp(self.h_offsets), _vp(self.h_col), self.Rb, self.Cb, M),
                            "mortar_sdd_blocks_per_wave_host")
            if len(self._sdd) > 256:                        # many token counts seen: keep the plans, forget the choices
                self._sdd = {k: v for k, v in self._sdd.items() if not isinstance(k, tuple)}
            self._sdd[("M", M)] = nb
        if nb not in self._sdd:
            n = _lib.check(L.mortar_sdd_plan_host(_vp(self.h_offsets), _vp(self.h_col), self.Rb, self.Cb, nb, None, 0),
                           "mortar_sdd_plan_host")
            plan = np.empty(n, dtype=np.int32)
            _lib.check(L.mortar_sdd_plan_host(_vp(self.h_offsets), _vp(self.h_col), self.Rb, self.Cb, nb, _vp(plan), n),
                       "mortar_sdd_plan_host")
            self._sdd[nb] = (torch.from_numpy(plan).to(self.device), int(plan[0]))
        return (*self._sdd[nb], nb)

    def sched(self, rows_per_unit: int) -> torch.Tensor:
        """Device schedule (mortar_schedule_host over the balanced unit order) for plain (1) or gate/up (2) units."""
        if rows_per_unit not in self._scheds:
            o = unit_order(self.h_offsets, self.Rb, rows_per_unit, snake=self.nseg > 1)
            if self.nseg > 1:
                o = unit_order_segments(self.h_row_desc, self.Rb, self.nseg, rows_per_unit, o)
            sc = schedule(self.h_row_desc, self.Rb, self.nseg, rows_per_unit, o)
            self._scheds[rows_per_unit] = torch.from_numpy(sc).to(self.device)
        return self._scheds[rows_per_unit]

    def worklist(self, rows_per_unit: int, kseg: int, max_blocks: int):
        key = (rows_per_unit, kseg, max_blocks)
        if key not in self._worklists:
            ent, ns, rs = decode_worklist(self.h_offsets, self.h_col, self.Rb, self.Cb, rows_per_unit, kseg, max_blocks)
            self._worklists[key] = (torch.from_numpy(ent).to(self.device), ns, torch.from_numpy(rs).to(self.device), ent)
        return self._worklists[key]

    @property
    def weight_bytes(self) -> int:
        """Algorithmic weight-side bytes: 64 B codes + 4 B scale + 2 B column id per block + 4 B per row pointer."""
        return self.nnz * 70 + 4 * (self.Rb + 1)

    def clone_weights(self) -> "MortarPack":
        """A second resident copy (own device buffers and schedules) of the same matrix."""
        import copy
        c = copy.copy(self)
        for name in ("codes", "sdup", "col", "row_ptr", "row_desc", "codes_o", "sd_o", "col_o", "codes4_o", "scales_f32"):
            if getattr(self, name) is not None:
                setattr(c, name, getattr(self, name).clone())
        c._scheds = {k: v.clone() for k, v in self._scheds.items()}
        c._worklists = {k: (v[0].clone(), v[1], v[2].clone(), v[3]) for k, v in self._worklists.items()}
        c._transposed, c._dview = None, {}      # the clone builds its own views
        c.struct = c._make_struct()
        c.ref = C.byref(c.struct)
        return c
