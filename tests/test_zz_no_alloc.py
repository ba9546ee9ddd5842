"""The allocation-free decode GEMV (mortar_gemv_bf16_noalloc) against mortar_gemv_bf16, through the C-ABI: same bits,
on two calls in a row (the second smaller, so it finds the first call's partial sums in the shared buffer), with and
without the fused SwiGLU, gather flags and gates; and the size limit is refused with a clear error."""
import ctypes as C

import numpy as np
import pytest
import torch

from mortar_amd import _lib, ops, synth
from oracle import mortar_oracle as O
from util import assert_close_bf16, to_dev, to_np

pytestmark = pytest.mark.gpu


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _call(noalloc, W, x, swiglu, max_blocks, gates=None, row_act=None, col_act=None):
    """One call through the C-ABI; returns (y, nslots).  The caller workspace of the existing entry point is poisoned
    with NaN first so that a slot read before it is written would show."""
    L = _lib.lib()
    B = x.shape[0]
    kseg = ops._kseg_for(W, B)
    ent, nslots, row_slots, _ = W.worklist(2 if swiglu else 1, kseg, max_blocks)
    nout = W.out_features // 2 if swiglu else W.out_features
    y = torch.full((B, nout), float("nan"), dtype=torch.bfloat16, device=x.device)
    st = C.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    ncl, ldg = (gates.shape[1], gates.stride(0)) if gates is not None else (0, 0)
    tail = (_p(gates), ncl, ldg, _p(row_act), row_act.stride(0) if row_act is not None else 0,
            _p(col_act), col_act.stride(0) if col_act is not None else 0, st)
    head = (W.ref, _p(ent), ent.shape[0], nslots, _p(row_slots), kseg, 1 if swiglu else 0, _p(x), B, x.stride(0), _p(y), y.stride(0))
    if noalloc:
        rc = L.mortar_gemv_bf16_noalloc(*head, *tail)
    else:
        part = torch.full((max(nslots, 1), B, W.out_features), float("nan"), dtype=torch.float32, device=x.device)
        rc = L.mortar_gemv_bf16(*head, _p(part), *tail)
    _lib.check(rc, "gemv")
    return y, nslots


def test_noalloc_gemv_matches_the_workspace_form(dev):
    spec = synth.synth_mlp(512, 16 * 96, 0.25, seed=500, zipf_s=1.2)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    small = synth.to_pack(synth.synth_matrix(16 * 6, 16 * 20, 0.5, seed=501), dev)
    # first call: 16 streams, gate_up with SwiGLU, rows split into several partial slots
    x16 = to_dev(synth.synth_x(16, 512, 502), dev)
    lg = torch.from_numpy(synth.synth_logits(16, 16, 503)).to(dev)
    gates, _ = ops.remoe_gates(lg, 5)
    ract, cact = ops.route_flags(gates, 16 * 96)
    want, ns = _call(False, Wgu, x16, True, 3, gates, ract, None)
    assert ns > 1
    got, _ = _call(True, Wgu, x16, True, 3, gates, ract, None)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    ref = O.swiglu_mlp(to_np(x16), spec["gate_up"], spec["down"], gates=gates.cpu().numpy())
    assert_close_bf16(to_np(got), ref["h"], "noalloc h", ulps=4)
    # second call, smaller in every way (3 streams, a small matrix, other slot count): the buffer still holds the
    # first call's partial sums
    x3 = to_dev(synth.synth_x(3, 16 * 20, 504), dev)
    want2, ns2 = _call(False, small, x3, False, 2)
    got2, _ = _call(True, small, x3, False, 2)
    assert ns2 > 1 and torch.equal(got2.view(torch.int16), want2.view(torch.int16))
    # third: down after gate_up (plain mode, wide K), and a single-slot list that needs no partial sums at all
    h = got
    want3, ns3 = _call(False, Wdn, h, False, 8, None, None, cact)
    got3, _ = _call(True, Wdn, h, False, 8, None, None, cact)
    assert ns3 > 1 and torch.equal(got3.view(torch.int16), want3.view(torch.int16))
    assert_close_bf16(to_np(got3), ref["y"], "noalloc y", ulps=8)
    want4, ns4 = _call(False, small, x3, False, 1 << 20)
    got4, _ = _call(True, small, x3, False, 1 << 20)
    assert ns4 == 1 and torch.equal(got4.view(torch.int16), want4.view(torch.int16))


def test_noalloc_gemv_refuses_what_does_not_fit(dev):
    L = _lib.lib()
    cap = int(L.mortar_gemv_noalloc_max_floats())
    assert cap == 1 << 20
    W = synth.to_pack(synth.synth_matrix(16 * 704, 16 * 32, 0.25, seed=510), dev)      # 11264 outputs
    x = to_dev(synth.synth_x(64, 16 * 32, 511), dev)
    _, ns = _call(False, W, x, False, 2)
    assert ns * 64 * W.out_features > cap
    with pytest.raises((ValueError, RuntimeError), match="exceed the built-in buffer"):
        _call(True, W, x, False, 2)
    y, _ = _call(True, W, x[:16], False, 2)                                            # 4 * 16 * 11264 floats fit
    w, _ = _call(False, W, x[:16], False, 2)
    assert torch.equal(y.view(torch.int16), w.view(torch.int16))
