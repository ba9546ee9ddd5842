"""Operator-level entry points: the reference's sparse-backend and decode-kernel call signatures, served by
the HIP library.  Every function requires tensors on a ROCm device; there is no CPU path."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from . import _lib
from .pack import BLK, BcsrTopology, MortarPack


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: Tensor):
    """The current stream of t's device as a raw handle (ctypes converts the int to void*)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(t: Tensor, what: str):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensor must live on a ROCm device (the MORTAR runtime has no CPU path)")


def _bf16_2d(x: Tensor, what: str) -> Tensor:
    _need_gpu(x, what)
    if x.dtype != torch.bfloat16:
        raise TypeError(f"{what}: expected bfloat16, got {x.dtype}")
    if x.dim() != 2:
        raise ValueError(f"{what}: expected a 2-D tensor")
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    return x


def _p(t):
    return t.data_ptr() if t is not None else None


# ----------------------------------------------------------------------------- prefill


def spmm(x: Tensor, W: MortarPack, out: Tensor | None = None, active: Tensor | None = None) -> Tensor:
    """y[M, out] = x[M, in] @ W^T, bf16 -> bf16, fp32 accumulate.  ``active`` (uint8 [M, n_clusters]) zeroes
    the input elements of inactive clusters on load."""
    x = _bf16_2d(x, "spmm")
    M = x.shape[0]
    if x.shape[1] != W.in_features:
        raise ValueError(f"spmm: x has {x.shape[1]} features, matrix expects {W.in_features}")
    y = out if out is not None else torch.empty((M, W.out_features), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    L = _lib.lib()
    sched = W.sched(1)
    if active is None:
        rc = L.mortar_spmm_bf16(W.ref, _p(sched), _p(x), M, x.stride(0), _p(y), y.stride(0), _stream(x))
    else:
        if active.dtype != torch.uint8 or not active.is_contiguous():
            raise TypeError("spmm: active must be a contiguous uint8 tensor")
        rc = L.mortar_spmm_bf16_masked(W.ref, _p(sched), _p(x), M, x.stride(0), _p(y), y.stride(0),
                                       _p(active), active.shape[1], _stream(x))
    _lib.check(rc, "mortar_spmm_bf16")
    return y


def dds_values(x: Tensor, data: Tensor, T: BcsrTopology, out: Tensor | None = None) -> Tensor:
    """y[M, out] = x[M, in] @ W^T for W given as stored bf16 block values ``data`` [nnz, 16, 16] on the topology ``T``:
    the arithmetic of the reference's stk_dds (custom_ops.py:35-56) for any block values, nothing quantised."""
    x = _bf16_2d(x, "dds_values")
    _need_gpu(data, "dds_values")
    if data.dtype != torch.bfloat16 or tuple(data.shape) != (T.nnz, BLK, BLK) or not data.is_contiguous():
        raise TypeError(f"dds_values: data must be a contiguous bfloat16 [{T.nnz}, 16, 16] tensor")
    if x.shape[1] != T.in_features:
        raise ValueError(f"dds_values: x has {x.shape[1]} features, matrix expects {T.in_features}")
    M = x.shape[0]
    y = out if out is not None else torch.empty((M, T.out_features), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    if T.nnz == 0:
        return y.zero_()
    rc = _lib.lib().mortar_dds_values_bf16(_p(T.row_ptr), _p(T.col), _p(T.seg_ptr), _p(data), T.Rb, T.Cb, T.nnz, _p(x), M,
                                           x.stride(0), _p(y), y.stride(0), _stream(x))
    _lib.check(rc, "mortar_dds_values_bf16")
    return y


def spmm_hc_post(x: Tensor, W: MortarPack, carrier: Tensor, hres: Tensor, hpost: Tensor, term: Tensor | None = None,
                 active: Tensor | None = None, out: Tensor | None = None) -> Tensor:
    """`down` with the hyper-connection POST write in its epilogue (decode batches, M <= 64): returns
    out[t, i] = sum_j hres[t, i, j] * carrier[t, j] + hpost[t, i] * (x W^T)[t] (+ term[t]); carrier / out [M, n, out_features]
    in bf16 or fp32, hres fp32 [M, n, n], hpost fp32 [M, n], term [M, out_features] of the carrier's dtype.  The
    reference runs the MLP, stores y, then launches _hc_post_fwd_kernel (engine.py:996-1001, 1052-1060)."""
    x = _bf16_2d(x, "spmm_hc_post")
    M = x.shape[0]
    if x.shape[1] != W.in_features:
        raise ValueError(f"spmm_hc_post: x has {x.shape[1]} features, matrix expects {W.in_features}")
    if carrier.dtype not in (torch.bfloat16, torch.float32) or carrier.dim() != 3 or not carrier.is_contiguous():
        raise TypeError("spmm_hc_post: carrier must be a contiguous bf16 or fp32 [M, n, out_features] tensor")
    _need_gpu(carrier, "spmm_hc_post")
    n = carrier.shape[1]
    if carrier.shape[0] != M or carrier.shape[2] != W.out_features:
        raise ValueError(f"spmm_hc_post: carrier is {tuple(carrier.shape)}, expected ({M}, n, {W.out_features})")
    for name, t, shape in (("hres", hres, (M, n, n)), ("hpost", hpost, (M, n))):
        if t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous():
            raise TypeError(f"spmm_hc_post: {name} must be contiguous float32 {shape}")
    if term is not None and (term.dtype != carrier.dtype or tuple(term.shape) != (M, W.out_features) or not term.is_contiguous()):
        raise TypeError("spmm_hc_post: term must be contiguous [M, out_features] of the carrier's dtype")
    res = out if out is not None else torch.empty_like(carrier)
    if M == 0:
        return res
    if active is not None and (active.dtype != torch.uint8 or not active.is_contiguous()):
        raise TypeError("spmm_hc_post: active must be a contiguous uint8 tensor")
    rc = _lib.lib().mortar_spmm_hc_post(W.ref, _p(W.sched(1)), _p(x), M, x.stride(0), _p(carrier),
                                        int(carrier.dtype == torch.float32), n, _p(hres), _p(hpost), _p(term), _p(res),
                                        _p(active), active.shape[1] if active is not None else 0, _stream(x))
    _lib.check(rc, "mortar_spmm_hc_post")
    return res


def norm_fusable(W: MortarPack) -> bool:
    """True if gateup_swiglu can apply the RMSNorm in front of the MLP while it stages x (in_features <= 2048)."""
    return bool(_lib.lib().mortar_norm_fusable(W.Cb)) and W.nseg == 1


def gateup_swiglu(x: Tensor, W: MortarPack, gates: Tensor | None = None, route: tuple | None = None,
                  out: Tensor | None = None, norm: tuple | None = None) -> Tensor:
    """h[M, d_ff] = silu(gate) * up [* gates per cluster] with gate_up = W [2*d_ff, d_model].
    route = (tok_cnt, tok_list) from remoe_route switches on active-tile skipping.
    norm = (weight bf16 [d_model] or None, eps): x is RMS-normalised on the way in (same bits as rmsnorm() first);
    needs norm_fusable(W)."""
    x = _bf16_2d(x, "gateup_swiglu")
    M = x.shape[0]
    if W.Rb % 2:
        raise ValueError(f"gateup_swiglu: gate_up has an odd number of block-rows ({W.Rb}): not a [2*d_ff, d_model] matrix")
    d_ff = W.out_features // 2
    if x.shape[1] != W.in_features:
        raise ValueError(f"gateup_swiglu: x has {x.shape[1]} features, matrix expects {W.in_features}")
    h = out if out is not None else torch.empty((M, d_ff), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return h
    ncl = 0
    if gates is not None:
        if gates.dtype != torch.float32 or gates.dim() != 2 or not gates.is_contiguous() or gates.shape[0] != M:
            raise TypeError("gateup_swiglu: gates must be a contiguous float32 [M, n_clusters] tensor")
        ncl = gates.shape[1]
    cnt, lst = route if route is not None else (None, None)
    if norm is not None:
        nw, eps = norm
        if nw is not None:
            if nw.dtype != torch.bfloat16 or nw.dim() != 1 or nw.shape[0] != W.in_features or not nw.is_contiguous():
                raise TypeError("gateup_swiglu: norm weight must be a contiguous bfloat16 [in_features] tensor")
            _need_gpu(nw, "gateup_swiglu")
        rc = _lib.lib().mortar_norm_gateup_swiglu_bf16(W.ref, _p(W.sched(2)), _p(x), M, x.stride(0), _p(nw), float(eps),
                                                       _p(h), h.stride(0), _p(gates), ncl, _p(cnt), _p(lst), _stream(x))
        _lib.check(rc, "mortar_norm_gateup_swiglu_bf16")
        return h
    rc = _lib.lib().mortar_gateup_swiglu_bf16(W.ref, _p(W.sched(2)), _p(x), M, x.stride(0), _p(h),
                                              h.stride(0), _p(gates), ncl, _p(cnt), _p(lst), _stream(x))
    _lib.check(rc, "mortar_gateup_swiglu_bf16")
    return h


def mlp(x: Tensor, Wgu: MortarPack, Wdn: MortarPack, gates: Tensor | None = None, norm: tuple | None = None,
        out: Tensor | None = None, hidden: Tensor | None = None, phase: int = 0) -> Tensor:
    """y[M, d_model] = down(silu(gate) * up [* gates per cluster]), gate_up applied to x or (``norm`` = (weight or None,
    eps), needs norm_fusable(Wgu)) to RMSNorm(x): _SwiGLUMortar.forward (transformer.py:402-431) in two launches.  Same bits
    as gateup_swiglu followed by spmm; the hidden activations stay in a workspace whose layout the library chooses (tile
    order for prefill-sized calls).  ``hidden``: a uint8 workspace of hidden_bytes(M, d_ff) to reuse across calls;
    ``phase`` 1 / 2 run only the first / second launch."""
    x = _bf16_2d(x, "mlp")
    M = x.shape[0]
    if x.shape[1] != Wgu.in_features:
        raise ValueError(f"mlp: x has {x.shape[1]} features, gate_up expects {Wgu.in_features}")
    if Wgu.Rb % 2 or Wgu.out_features != 2 * Wdn.in_features:
        raise ValueError(f"mlp: gate_up [{Wgu.out_features}, {Wgu.in_features}] and down [{Wdn.out_features}, {Wdn.in_features}] do not chain")
    d_ff = Wdn.in_features
    y = out if out is not None else torch.empty((M, Wdn.out_features), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    L = _lib.lib()
    need = int(L.mortar_mlp_hidden_bytes(M, d_ff))
    if hidden is None:
        hidden = torch.empty(need, dtype=torch.uint8, device=x.device)
    elif hidden.dtype != torch.uint8 or not hidden.is_contiguous() or hidden.numel() < need or hidden.device != x.device:
        raise ValueError(f"mlp: hidden must be a contiguous uint8 workspace of at least {need} bytes on {x.device}")
    ncl = 0
    if gates is not None:
        if gates.dtype != torch.float32 or gates.dim() != 2 or not gates.is_contiguous() or gates.shape[0] != M:
            raise TypeError("mlp: gates must be a contiguous float32 [M, n_clusters] tensor")
        ncl = gates.shape[1]
    nw, eps = (None, 0.0)
    if norm is not None:
        nw, eps = norm
        if nw is not None:
            if nw.dtype != torch.bfloat16 or nw.dim() != 1 or nw.shape[0] != Wgu.in_features or not nw.is_contiguous():
                raise TypeError("mlp: norm weight must be a contiguous bfloat16 [in_features] tensor")
            _need_gpu(nw, "mlp")
    rc = L.mortar_mlp_bf16(Wgu.ref, _p(Wgu.sched(2)), Wdn.ref, _p(Wdn.sched(1)), _p(x), M, x.stride(0), int(norm is not None),
                           _p(nw), float(eps), _p(gates), ncl, _p(hidden), _p(y), y.stride(0), int(phase), _stream(x))
    _lib.check(rc, "mortar_mlp_bf16")
    return y


def mlp_hidden_bytes(M: int, d_ff: int) -> int:
    return int(_lib.lib().mortar_mlp_hidden_bytes(int(M), int(d_ff)))


# ----------------------------------------------------------------------------- ReMoE


def remoe_gates(logits: Tensor, k: int) -> tuple[Tensor, Tensor]:
    """(gates fp32 [M, n], active uint8 [M, n]) from fp32 logits: TileRouter.forward steps 5-8."""
    _need_gpu(logits, "remoe_gates")
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise TypeError("remoe_gates: logits must be float32 [M, n]")
    logits = logits.contiguous()
    M, n = logits.shape
    gates = torch.empty_like(logits)
    active = torch.empty((M, n), dtype=torch.uint8, device=logits.device)
    if M:
        _lib.check(_lib.lib().mortar_remoe_gates(_p(logits), M, n, int(k), _p(gates), _p(active), _stream(logits)),
                   "mortar_remoe_gates")
    return gates, active


ROUTER_MAX_TOKENS = 64
DECODE_MAX_ROWS = 64      # rows up to which a call runs on the 4- / 16-token decode tiles


def router_fused(x: Tensor, wq: Tensor, iter_vec: Tensor | None, ln_w: Tensor, ln_b: Tensor, ln_eps: float,
                 ka: Tensor, kb: Tensor, bias: Tensor, k: int, want_logits: bool = False):
    """Decode-side TileRouter in two launches (projection, then LayerNorm + product keys + gating tail).
    x [B <= 64, d] bf16 or fp32; all parameters fp32.  -> (gates fp32 [B, n], active uint8 [B, n][, logits])."""
    _need_gpu(x, "router_fused")
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("router_fused: x must be a 2-D bfloat16 or float32 tensor")
    if x.stride(1) != 1:
        x = x.contiguous()
    B, d = x.shape
    n, nsk = bias.numel(), ka.shape[0]
    for name, t, shp in (("wq", wq, (d, d)), ("ln_w", ln_w, (d,)), ("ln_b", ln_b, (d,)), ("ka", ka, (nsk, d // 2)),
                         ("kb", kb, (nsk, d // 2)), ("bias", bias, (n,))) + ((("iter_vec", iter_vec, (d,)),) if iter_vec is not None else ()):
        if t.dtype != torch.float32 or tuple(t.shape) != shp or not t.is_contiguous() or t.device != x.device:
            raise TypeError(f"router_fused: {name} must be a contiguous float32 {shp} tensor on {x.device}")
    qv = torch.empty((B, d), dtype=torch.float32, device=x.device)
    gates = torch.empty((B, n), dtype=torch.float32, device=x.device)
    active = torch.empty((B, n), dtype=torch.uint8, device=x.device)
    logits = torch.empty((B, n), dtype=torch.float32, device=x.device) if want_logits else None
    if B:
        rc = _lib.lib().mortar_router_bf16(_p(x), int(x.dtype == torch.float32), B, d, x.stride(0), _p(wq), _p(iter_vec),
                                           _p(ln_w), _p(ln_b), float(ln_eps), _p(ka), _p(kb), nsk, _p(bias), n, int(k),
                                           _p(qv), _p(logits), _p(gates), _p(active), _stream(x))
        _lib.check(rc, "mortar_router_bf16")
    return (gates, active, logits) if want_logits else (gates, active)


def router_tail(qv: Tensor, iter_vec: Tensor | None, ln_w: Tensor, ln_b: Tensor, ln_eps: float, ka: Tensor, kb: Tensor,
                bias: Tensor, k: int, want_logits: bool = False):
    """TileRouter.forward steps 2-8 in one launch on the projected query qv = x Wq^T (fp32 [N, d], any N): LayerNorm of
    qv + iter_vec, sub-key scores, product-key logits, gating tail.  The projection itself is a dense GEMM and stays with
    the library.  -> (gates fp32 [N, n], active uint8 [N, n][, logits])."""
    _need_gpu(qv, "router_tail")
    if qv.dim() != 2 or qv.dtype != torch.float32:
        raise TypeError("router_tail: qv must be a 2-D float32 tensor")
    if qv.stride(1) != 1 or qv.stride(0) % 4 or qv.data_ptr() % 16:
        qv = qv.contiguous()
    N, d = qv.shape
    n, nsk = bias.numel(), ka.shape[0]
    for name, t, shp in (("ln_w", ln_w, (d,)), ("ln_b", ln_b, (d,)), ("ka", ka, (nsk, d // 2)), ("kb", kb, (nsk, d // 2)),
                         ("bias", bias, (n,))) + ((("iter_vec", iter_vec, (d,)),) if iter_vec is not None else ()):
        if t.dtype != torch.float32 or tuple(t.shape) != shp or not t.is_contiguous() or t.device != qv.device:
            raise TypeError(f"router_tail: {name} must be a contiguous float32 {shp} tensor on {qv.device}")
    gates = torch.empty((N, n), dtype=torch.float32, device=qv.device)
    active = torch.empty((N, n), dtype=torch.uint8, device=qv.device)
    logits = torch.empty((N, n), dtype=torch.float32, device=qv.device) if want_logits else None
    if N:
        rc = _lib.lib().mortar_router_tail_f32(_p(qv), N, d, qv.stride(0), _p(iter_vec), _p(ln_w), _p(ln_b), float(ln_eps),
                                               _p(ka), _p(kb), nsk, _p(bias), n, int(k), _p(logits), _p(gates), _p(active),
                                               _stream(qv))
        _lib.check(rc, "mortar_router_tail_f32")
    return (gates, active, logits) if want_logits else (gates, active)


def route_tile(W: MortarPack, M: int = 0) -> int:
    """Token tile of the routed gate_up kernels for M rows against this matrix (the tile remoe_route must use);
    0 when the matrix is too wide for routed skipping (use the dense gated call)."""
    return int(_lib.lib().mortar_route_tile(W.Cb, int(M)))


def remoe_route(active: Tensor, tile: int) -> tuple[Tensor, Tensor]:
    """Per (token tile, cluster): count and ascending list of the tile-local indices of active tokens."""
    _need_gpu(active, "remoe_route")
    if active.dtype != torch.uint8 or active.dim() != 2 or not active.is_contiguous():
        raise TypeError("remoe_route: active must be a contiguous uint8 [M, n] tensor")
    M, n = active.shape
    nt = -(-M // tile)
    cnt = torch.empty((nt, n), dtype=torch.int32, device=active.device)
    lst = torch.empty((nt, n, tile), dtype=torch.uint8, device=active.device)
    _lib.check(_lib.lib().mortar_remoe_route(_p(active), M, n, tile, _p(cnt), _p(lst), _stream(active)),
               "mortar_remoe_route")
    return cnt, lst


def route_flags(gates: Tensor, d_ff: int, row_act: Tensor | None = None, col_act: Tensor | None = None):
    """Decode gather flags (reference route_flags with blk = 16): row_act int32 [B, 2*d_ff/16],
    col_act int32 [B, d_ff/16]; out buffers may be sliced views of a wider scratch."""
    _need_gpu(gates, "route_flags")
    if gates.dtype != torch.float32 or gates.dim() != 2 or gates.stride(1) != 1:
        raise TypeError("route_flags: gates must be float32 [B, n_clusters] with unit inner stride")
    B, ncl = gates.shape
    nc = d_ff // BLK
    if row_act is None:
        row_act = torch.empty((B, 2 * nc), dtype=torch.int32, device=gates.device)
    if col_act is None:
        col_act = torch.empty((B, nc), dtype=torch.int32, device=gates.device)
    _lib.check(_lib.lib().mortar_route_flags(_p(gates), B, ncl, gates.stride(0), d_ff, _p(row_act), row_act.stride(0),
                                             _p(col_act), col_act.stride(0), _stream(gates)), "mortar_route_flags")
    return row_act, col_act


def swiglu(gu: Tensor, out: Tensor | None = None) -> Tensor:
    """h = silu(gate) * up from a stored gate_up output gu [M, 2*d_ff] (training form; inference fuses this into gate_up)."""
    gu = _bf16_2d(gu, "swiglu")
    M, d_ff = gu.shape[0], gu.shape[1] // 2
    if gu.shape[1] % 16:
        raise ValueError("swiglu: gate_up width must be a multiple of 16")
    h = out if out is not None else torch.empty((M, d_ff), dtype=torch.bfloat16, device=gu.device)
    _lib.check(_lib.lib().mortar_swiglu_bf16(_p(gu), gu.stride(0), M, d_ff, _p(h), h.stride(0), _stream(gu)), "mortar_swiglu_bf16")
    return h


def swiglu_backward(gu: Tensor, dh: Tensor) -> Tensor:
    """d(gate_up output) [M, 2*d_ff] from the stored gate_up output and dh [M, d_ff]."""
    gu, dh = _bf16_2d(gu, "swiglu_backward"), _bf16_2d(dh, "swiglu_backward")
    M, d_ff = gu.shape[0], gu.shape[1] // 2
    if gu.shape[1] % 16 or tuple(dh.shape) != (M, d_ff):
        raise ValueError(f"swiglu_backward: gu {tuple(gu.shape)} / dh {tuple(dh.shape)} do not match")
    dgu = torch.empty_like(gu)
    _lib.check(_lib.lib().mortar_swiglu_backward_bf16(_p(gu), gu.stride(0), _p(dh), dh.stride(0), M, d_ff, _p(dgu),
                                                      dgu.stride(0), _stream(gu)), "mortar_swiglu_backward_bf16")
    return dgu


def sdd(a: Tensor, b: Tensor, W: MortarPack, out: Tensor | None = None, blocks_per_wave: int | None = None) -> Tensor:
    """Weight gradient on W's topology: out[j] = a[:, rows of block j]^T @ b[:, columns of block j], bf16 [nnz,16,16]
    (reference stk_sdd_at_b; for y = x W^T pass a = dY [M, out_features], b = x [M, in_features]).
    `blocks_per_wave` picks the kernel's group size instead of the library's choice for this topology and M."""
    a, b = _bf16_2d(a, "sdd"), _bf16_2d(b, "sdd")
    if a.shape[0] != b.shape[0] or a.shape[1] != W.out_features or b.shape[1] != W.in_features:
        raise ValueError(f"sdd: a {tuple(a.shape)} / b {tuple(b.shape)} do not match the matrix [{W.out_features}, {W.in_features}]")
    if a.stride(0) % 8 or a.data_ptr() % 16:
        a = a.contiguous()
    if b.stride(0) % 8 or b.data_ptr() % 16:
        b = b.contiguous()
    plan, n_wg, nb = W.sdd_plan(a.shape[0], blocks_per_wave)
    if out is None:
        out = torch.empty((W.nnz, BLK, BLK), dtype=torch.bfloat16, device=a.device)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (W.nnz, BLK, BLK) or not out.is_contiguous():
        raise TypeError("sdd: out must be a contiguous bfloat16 [nnz, 16, 16] tensor")
    ws = _lib.check(_lib.lib().mortar_sdd_workspace_bytes(n_wg, W.nnz, nb, a.shape[0]), "mortar_sdd_workspace_bytes")
    acc = torch.empty(ws // 4, dtype=torch.float32, device=a.device)
    _lib.check(_lib.lib().mortar_sdd_bf16(_p(plan), n_wg, nb, W.Rb, W.Cb, W.nnz, _p(a), a.stride(0), _p(b), b.stride(0),
                                          a.shape[0], _p(acc), _p(out), _stream(a)), "mortar_sdd_bf16")
    return out


# ----------------------------------------------------------------------------- decode


def _kseg_for(W: MortarPack, B: int) -> int:
    """Block-columns per K segment so that the staged activations fit in 64 KiB of LDS."""
    mt = 16 if B <= 16 else (32 if B <= 32 else 64)
    units = (64 * 1024) // ((mt + 1) * 16)        # 16-byte units = column halves
    return max(2, min(W.Cb, units // 2))


def gemv(x: Tensor, W: MortarPack, swiglu_out: bool = False, gates: Tensor | None = None,
         row_act: Tensor | None = None, col_act: Tensor | None = None, max_blocks: int | None = None,
         out: Tensor | None = None, flags_from_gates: bool = True) -> Tensor:
    """Decode GEMV for B <= 64 streams: y = x W^T (bf16), or with swiglu_out the fused silu(g)*u[*gates].
    Without gather flags the batch goes to the small-tile SpMM kernels (one pass over the weights); with
    row_act / col_act (or an explicit max_blocks split) it runs the work-list kernel that honours them, per stream.
    ``flags_from_gates``: row_act is route_flags(gates) of this very call, as the reference engine passes it
    (engine.py:984-994); the gated gate_up then needs no flags (a gate of 0 zeroes what the flag would).  Pass False
    for flags of any other origin: they are then applied as given."""
    x = _bf16_2d(x, "gemv")
    B = x.shape[0]
    if not 1 <= B <= 64:
        raise ValueError(f"gemv: batch {B} outside 1..64 (use the prefill path)")
    if x.shape[1] != W.in_features:
        raise ValueError(f"gemv: x has {x.shape[1]} features, matrix expects {W.in_features}")
    # rows so wide that not even a 4-token tile of all K fits in LDS (in_features > 19904) run 2-token tiles up to 4
    # rows; beyond that they go to the work-list kernel, which splits K over workgroups and combines partial sums
    rt1 = getattr(W, "_route_tile_1", None)
    if rt1 is None:
        rt1 = W._route_tile_1 = route_tile(W, 1)
    # gate_up with gates: the row flags add nothing there (the gated kernel leaves out the units whose cluster is off for
    # every stream and stores their zeros; every other unit is computed and gated per stream, as the work list does)
    if swiglu_out and gates is not None and col_act is None and max_blocks is None and rt1 != 0 and flags_from_gates:
        row_act = None
    if row_act is None and col_act is None and max_blocks is None and (rt1 != 0 or (B <= 4 and not swiglu_out)):
        if swiglu_out:
            return gateup_swiglu(x, W, gates=gates.contiguous() if gates is not None else None, out=out)
        return spmm(x, W, out=out)
    rpu = 2 if swiglu_out else 1
    kseg = _kseg_for(W, B)
    if max_blocks is None:
        max_blocks = 1 << 20                       # whole row (per segment) in one entry
    ent, nslots, row_slots, _ = W.worklist(rpu, kseg, max_blocks)
    nout = W.out_features // 2 if swiglu_out else W.out_features
    y = out if out is not None else torch.empty((B, nout), dtype=torch.bfloat16, device=x.device)
    part = None
    if nslots > 1:
        part = torch.empty((nslots, B, W.out_features), dtype=torch.float32, device=x.device)
    ncl, ldg = 0, 0
    if gates is not None:
        if gates.dtype != torch.float32 or gates.stride(1) != 1:
            raise TypeError("gemv: gates must be float32 with unit inner stride")
        ncl, ldg = gates.shape[1], gates.stride(0)
    for f in (row_act, col_act):
        if f is not None and (f.dtype != torch.int32 or f.stride(1) != 1):
            raise TypeError("gemv: row_act / col_act must be int32 with unit inner stride")
    rc = _lib.lib().mortar_gemv_bf16(
        W.ref, _p(ent), ent.shape[0], nslots, _p(row_slots), kseg, 1 if swiglu_out else 0,
        _p(x), B, x.stride(0), _p(y), y.stride(0), _p(part), _p(gates), ncl, ldg,
        _p(row_act), row_act.stride(0) if row_act is not None else 0,
        _p(col_act), col_act.stride(0) if col_act is not None else 0, _stream(x))
    _lib.check(rc, "mortar_gemv_bf16")
    return y


def gemv_f32(x: Tensor, W: MortarPack, swiglu_x: bool = False, swiglu_out: bool = False, gates: Tensor | None = None,
             row_act: Tensor | None = None, col_act: Tensor | None = None, max_blocks: int | None = None,
             out: Tensor | None = None) -> Tensor:
    """Decode GEMV in the reference engine's arithmetic (fp32 activations, exact products, fp32 sums, fp32 scale after
    the block sum, fp32 out): the reference's mortar_gemv (fused_decode_step.py:1502-1547).  ``swiglu_x``: x is the
    gate_up output [B, 2 * in_features] and silu(g) * u is applied on load; ``swiglu_out``: W is gate_up and the result
    is silu(g) * u [* gates]."""
    _need_gpu(x, "gemv_f32")
    if x.dtype != torch.float32 or x.dim() != 2:
        raise TypeError("gemv_f32: expected a float32 [B, features] tensor")
    if x.stride(1) != 1:
        x = x.contiguous()
    B = x.shape[0]
    if not 1 <= B <= 64:
        raise ValueError(f"gemv_f32: batch {B} outside 1..64")
    need = W.in_features * (2 if swiglu_x else 1)
    if x.shape[1] != need:
        raise ValueError(f"gemv_f32: x has {x.shape[1]} features, expected {need}")
    if W.scales_f32 is None:
        raise ValueError("gemv_f32: the pack holds no scales yet (requantize it first)")
    if swiglu_out and W.Rb % 2:
        raise ValueError("gemv_f32: gate_up has an odd number of block-rows")
    mt = 16 if B <= 16 else (32 if B <= 32 else 64)
    kseg = max(2, min(W.Cb, (48 * 1024) // ((mt + 1) * 16) // 2))       # three term planes of at most 48 KiB each
    ent, nslots, row_slots, _ = W.worklist(2 if swiglu_out else 1, kseg, max_blocks if max_blocks is not None else 1 << 20)
    nout = W.out_features // 2 if swiglu_out else W.out_features
    y = out if out is not None else torch.empty((B, nout), dtype=torch.float32, device=x.device)
    sc = W.scales_f32
    sc_one = sc.numel() == 1
    L = _lib.lib()
    # one scale, no explicit split: the SpMM kernels run the product (flags zero what the work list would skip)
    fast = sc_one and max_blocks is None
    ws = _lib.check(L.mortar_gemv_f32_workspace_bytes(W.ref, B, nslots), "mortar_gemv_f32_workspace_bytes")
    part = torch.empty(ws // 4, dtype=torch.float32, device=x.device) if (nslots > 1 or fast) else None
    if fast and ((B > 1 and x.stride(0) % 4) or x.data_ptr() % 16):       # the split kernel reads 16-byte words
        x = x.clone(memory_format=torch.contiguous_format)
    ncl, ldg = 0, 0
    if gates is not None:
        if gates.dtype != torch.float32 or gates.stride(1) != 1:
            raise TypeError("gemv_f32: gates must be float32 with unit inner stride")
        ncl, ldg = gates.shape[1], gates.stride(0)
    for f in (row_act, col_act):
        if f is not None and (f.dtype != torch.int32 or f.stride(1) != 1):
            raise TypeError("gemv_f32: row_act / col_act must be int32 with unit inner stride")
    rc = L.mortar_gemv_f32(
        W.ref, _p(sc), sc.numel(), _p(W.sched(1)) if fast else None, _p(ent), ent.shape[0], nslots, _p(row_slots), kseg,
        1 if swiglu_out else 0, 1 if swiglu_x else 0, _p(x), B, x.stride(0) if B > 1 else x.shape[1], _p(y), y.stride(0), _p(part),
        part.numel() * 4 if part is not None else 0, _p(gates), ncl, ldg,
        _p(row_act), row_act.stride(0) if row_act is not None else 0,
        _p(col_act), col_act.stride(0) if col_act is not None else 0, _stream(x))
    _lib.check(rc, "mortar_gemv_f32")
    return y


class LayerStack:
    """n layers of one shape (same Rb, Cb, K segments) whose small-M products run in ONE launch:
    y_l = x_l W_l^T, or with swiglu the fused silu(g)*u of gate_up W_l.  The inputs and outputs are fixed at
    construction (their device addresses go into a parameter table); run() may be called any number of times."""

    def __init__(self, packs: list[MortarPack], xs: list[Tensor], ys: list[Tensor], swiglu: bool = False):
        n = len(packs)
        if n == 0 or len(xs) != n or len(ys) != n:
            raise ValueError("LayerStack: need one input and one output per layer")
        xs = [_bf16_2d(x, "LayerStack") for x in xs]
        M = xs[0].shape[0]
        for x, y in zip(xs, ys):
            if x.shape != xs[0].shape or x.stride(0) != xs[0].stride(0) or y.stride(0) != ys[0].stride(0):
                raise ValueError("LayerStack: inputs / outputs must share shape and row stride")
            if y.dtype != torch.bfloat16 or not y.is_cuda:
                raise TypeError("LayerStack: outputs must be bfloat16 device tensors")
        L = _lib.lib()
        if M <= 4 and not swiglu:
            # products over several K segments (`down`) read their one-segment decode streams: one part and one padding to
            # octets per row (all layers or none: a launch takes one segment width)
            views = [p.decode_view(M) for p in packs]
            if all(v is not None for v in views):
                packs = views
        self.packs, self.xs, self.ys, self.swiglu, self.M, self.n = packs, xs, ys, int(bool(swiglu)), M, n
        self._structs = (_lib.BcsrStruct * n)(*[p.struct for p in packs])
        sp = (C.c_void_p * n)(*[p.sched(2 if swiglu else 1).data_ptr() for p in packs])
        xp = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
        yp = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
        self.table = torch.empty(int(L.mortar_stack_table_bytes(n)), dtype=torch.uint8, device=xs[0].device)
        _lib.check(L.mortar_stack_prepare(self.swiglu, n, self._structs, sp, xp, yp, M, xs[0].stride(0), ys[0].stride(0),
                                          _p(self.table), _stream(xs[0])), "mortar_stack_prepare")

    def run(self) -> list[Tensor]:
        _lib.check(_lib.lib().mortar_stack_run(self.swiglu, self.n, self._structs, self.M, _p(self.table),
                                               _stream(self.xs[0])), "mortar_stack_run")
        return self.ys


# ----------------------------------------------------------------------------- RMSNorm


def rmsnorm(x: Tensor, weight: Tensor | None = None, eps: float = 1e-6) -> Tensor:
    """bf16 RMSNorm over the last dim (attention.RMSNorm semantics: normalise in fp32, cast, scale)."""
    _need_gpu(x, "rmsnorm")
    shp = x.shape
    x2 = x.reshape(-1, shp[-1])
    if x2.dtype != torch.bfloat16:
        raise TypeError("rmsnorm: expected bfloat16")
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    w = None
    if weight is not None:
        w = weight.to(torch.bfloat16).contiguous()
    y = torch.empty_like(x2, memory_format=torch.contiguous_format)
    if x2.shape[0]:
        _lib.check(_lib.lib().mortar_rmsnorm_bf16(_p(x2), x2.shape[0], shp[-1], x2.stride(0), _p(w), float(eps), _p(y),
                                                  y.stride(0), _stream(x)), "mortar_rmsnorm_bf16")
    return y.reshape(shp)
