"""CPU tests of the host logic: C-ABI exports, device-format encoding, schedules, module state (no GPU compute)."""
import ctypes
import ctypes as C
import itertools
import os
import re

import numpy as np
import pytest
import torch

import mortar_amd
from mortar_amd import _lib, pack as P, synth
from oracle import mortar_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "mortar_hip.h")).read()
    code = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)                       # declarations only, not comments
    declared = set(re.findall(r"\b(mortar_[a-z0-9_]+)\s*\(", code))
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in mortar_hip.h but not exported"
    assert declared == set(_lib.EXPORTS)
    assert _lib.lib().mortar_abi_version() == 7


def test_encode_round_trip_and_bit_layout():
    rng = np.random.default_rng(0)
    codes = rng.integers(-1, 2, (9, 16, 16)).astype(np.int8)
    scale = rng.uniform(0.01, 0.1, 9).astype(np.float32)
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(codes), 9, scale)
    assert np.array_equal(P.decode_blocks(dw), codes)
    # the 8 columns of column half h are the top two bits (sign, non-zero) of the 8 nibbles of (w << 2h) & 0xCCCCCCCC,
    # in column order: as FP4 (E2M1) those nibbles are 0x4 = +2, 0xC = -2, 0 = 0
    for j, n, h, q in itertools.product((0, 8), (0, 7, 15), (0, 1), range(8)):
        w = int(dw[j * 16 + n])
        nib = ((((w << (2 * h)) & 0xFFFFFFFF) & 0xCCCCCCCC) >> (4 * q)) & 0xF
        assert {0x0: 0, 0x4: 1, 0xC: -1}[nib] == codes[j, n, 8 * h + q]
    # scale pattern: bf16 bits minus one 16-bit-float exponent step, in both halves
    s16 = O.bf16_bits(scale).astype(np.uint32) - 0x400
    assert np.array_equal(sdup, s16 | (s16 << 16))
    # multiplying the pattern (as 16-bit floats) by +-2 gives +-bf16(scale) bit-exactly
    half = (sdup & 0xFFFF).astype(np.uint16).view(np.float16)
    for sign in (2.0, -2.0):
        prod = (half.astype(np.float32) * np.float32(sign)).astype(np.float16).view(np.uint16)
        want = O.bf16_bits(scale) | (0x8000 if sign < 0 else 0)
        assert np.array_equal(prod, want)


def test_uniform_scale_is_detected():
    codes = np.ones((5, 16, 16), np.int8)
    L = _lib.lib()
    us = C.c_float(-1.0)
    _, sdup = P.encode_blocks(O.pack_ternary_codes(codes), 5, np.float32(0.0371))
    _lib.check(L.mortar_uniform_scale_host(P._vp(sdup), 5, C.byref(us)), "uniform")
    assert us.value == O.bf16_round(np.float32(0.0371))                  # the bf16 value the kernels multiply by
    _, sdup = P.encode_blocks(O.pack_ternary_codes(codes), 5, np.linspace(0.01, 0.1, 5).astype(np.float32))
    _lib.check(L.mortar_uniform_scale_host(P._vp(sdup), 5, C.byref(us)), "uniform")
    assert us.value == 0.0                                               # per-block scales
    _, sdup = P.encode_blocks(O.pack_ternary_codes(codes), 5, np.float32(0.0))
    _lib.check(L.mortar_uniform_scale_host(P._vp(sdup), 5, C.byref(us)), "uniform")
    assert us.value == 0.0


def test_encode_scalar_scale_and_errors():
    codes = np.ones((2, 16, 16), np.int8)
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(codes), 2, np.float32(0.05))
    assert sdup[0] == sdup[1]
    with pytest.raises(ValueError, match="outside"):
        P.encode_blocks(O.pack_ternary_codes(codes), 2, np.float32(1e38))
    with pytest.raises(ValueError, match="outside"):
        P.encode_blocks(O.pack_ternary_codes(codes), 2, np.float32(float("inf")))
    with pytest.raises(ValueError, match="scale_count"):
        P.encode_blocks(O.pack_ternary_codes(codes), 2, np.ones(3, np.float32))
    bad = O.pack_ternary_codes(codes).copy(); bad[5] = 0xFF
    with pytest.raises(ValueError, match="invalid 2-bit code"):
        P.encode_blocks(bad, 2, np.float32(1.0))
    dw0, sd0 = P.encode_blocks(O.pack_ternary_codes(codes), 2, np.float32(0.0))     # zero scale zeroes the block
    assert not dw0.any() and not sd0.any()


def test_validate_bcsr_rejects_bad_layouts():
    m = synth.synth_matrix(16 * 9, 16 * 50, 0.3, 3, zipf_s=1.2)
    P.validate_bcsr(m["offsets"], m["col_idx"], 9, 50)
    bad = m["col_idx"].copy(); bad[1] = bad[0]
    with pytest.raises(ValueError, match="ascending"):
        P.validate_bcsr(m["offsets"], bad, 9, 50)
    bad = m["col_idx"].copy(); bad[0] = 50
    with pytest.raises(ValueError, match="out of range"):
        P.validate_bcsr(m["offsets"], bad, 9, 50)
    off = m["offsets"].copy(); off[3] = off[2] - 1
    with pytest.raises(ValueError, match="decrease"):
        P.validate_bcsr(off, m["col_idx"], 9, 50)


@pytest.mark.parametrize("seg_cb", [50, 17, 7])
def test_octet_stream_holds_every_block_once(seg_cb):
    """Decoding the octet stream back (codes, scale pattern, column) reproduces the BCSR exactly, for one and
    for several K segments; padding blocks are all-zero."""
    Rb, Cb = 9, 50
    m = synth.synth_matrix(16 * Rb, 16 * Cb, 0.3, 3, zipf_s=1.2)
    nnz = int(m["offsets"][-1])
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(m["codes"]), nnz, m["scales"])
    desc, codes_o, sd_o, col_o = P.octet_layout(m["offsets"], Rb, Cb, seg_cb, dw, sdup, m["col_idx"])
    nseg = -(-Cb // seg_cb)
    desc = desc.reshape(nseg, Rb, 4)
    codes_o = codes_o.reshape(-1, 2, 16, 4); sd_o = sd_o.reshape(-1, 2, 4); col_o = col_o.reshape(-1, 2, 4)
    used = np.zeros(codes_o.shape[0], bool)
    for r in range(Rb):
        got = []
        for sg in range(nseg):
            g0, g1, nb, _ = desc[sg, r]
            assert g1 - g0 == -(-nb // 8) and not used[g0:g1].any()
            used[g0:g1] = True
            for b in range(8 * (g1 - g0)):
                g, t, s2 = g0 + b // 8, (b % 8) // 2, b % 2
                if b < nb:
                    got.append((int(col_o[g, s2, t]) + sg * seg_cb, int(sd_o[g, s2, t]), codes_o[g, s2, :, t].copy()))
                    assert 0 <= col_o[g, s2, t] < seg_cb
                else:
                    assert sd_o[g, s2, t] == 0 and not codes_o[g, s2, :, t].any()
        lo, hi = m["offsets"][r], m["offsets"][r + 1]
        assert [c for c, _, _ in got] == m["col_idx"][lo:hi].tolist()
        assert [s for _, s, _ in got] == sdup[lo:hi].tolist()
        assert np.array_equal(np.stack([w for _, _, w in got]), dw.reshape(-1, 16)[lo:hi])
    assert used.all()


def test_fp4_stream_holds_the_same_codes():
    """The 4-bit copy of the code stream decodes (FP4 E2M1: 0x4 = +2, 0xC = -2, 0 = 0, for codes +1 / -1 / 0) to the ternary codes of the
    block it mirrors, column 8h + q of row n in nibble q of dword (octet, 2s + h, n, t)."""
    Rb, Cb = 9, 50
    m = synth.synth_matrix(16 * Rb, 16 * Cb, 0.3, 5, zipf_s=1.2)
    nnz = int(m["offsets"][-1])
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(m["codes"]), nnz, m["scales"])
    desc, codes_o, _, _ = P.octet_layout(m["offsets"], Rb, Cb, 17, dw, sdup, m["col_idx"])
    c4 = P.fp4_stream(codes_o).reshape(-1, 2, 2, 16, 4)                       # octet, s, h, n, t
    assert c4.shape[0] * 128 == codes_o.size
    nib = (c4[..., None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF        # ..., q
    assert np.isin(nib, [0x0, 0x4, 0xC]).all()
    val = np.where(nib == 0x4, 1, np.where(nib == 0xC, -1, 0)).astype(np.int8)
    # the 2-bit stream's blocks, decoded with the library's own inverse: [octet, s, t] -> [16 rows, 16 cols]
    blocks = codes_o.reshape(-1, 2, 16, 4).transpose(0, 1, 3, 2).reshape(-1, 16)    # (octet, s, t) x n
    dec = np.empty((blocks.shape[0], 16, 16), np.int8)
    _lib.check(_lib.lib().mortar_decode_blocks_host(P._vp(np.ascontiguousarray(blocks)), blocks.shape[0], P._vp(dec)), "decode")
    dec = dec.reshape(-1, 2, 4, 16, 2, 8)                                      # octet, s, t, n, h, q
    assert np.array_equal(val, dec.transpose(0, 1, 4, 3, 2, 5))               # -> octet, s, h, n, t, q
    assert np.abs(dec).sum() == np.abs(m["codes"]).sum()                      # every kept code once, padding is zero


def test_unit_order_and_schedule():
    m = synth.synth_matrix(16 * 64, 16 * 40, 0.25, 4, zipf_s=1.2)
    nnz = int(m["offsets"][-1])
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(m["codes"]), nnz, m["scales"])
    desc, _, _, _ = P.octet_layout(m["offsets"], 64, 40, 17, dw, sdup, m["col_idx"])
    for rpu in (1, 2):
        o = P.unit_order(m["offsets"], 64, rpu)
        nu = 64 // rpu
        assert sorted(o.tolist()) == list(range(nu))
        cost = np.diff(m["offsets"])
        if rpu == 2:
            cost = cost[:nu] + cost[nu:]
        group = P.SCHED_GROUP
        loads = [cost[o[g:g + group]].sum() for g in range(0, nu, group)]
        naive = [cost[g:g + group].sum() for g in range(0, nu, group)]
        assert max(loads) <= max(naive)
        # groups hold the same units either way; without the snake every group is heaviest first, with it the odd
        # groups are reversed
        flat = P.unit_order(m["offsets"], 64, rpu, snake=False)
        for gi, g in enumerate(range(0, nu, group)):
            assert (np.diff(cost[flat[g:g + group]]) <= 0).all()
            assert flat[g:g + group].tolist() == (o[g:g + group][::-1] if gi % 2 else o[g:g + group]).tolist()
        sc = P.schedule(desc, 64, 3, rpu, o)                                            # [nu, nseg, rpu, 4]
        d3 = desc.reshape(3, 64, 4)
        for pos in (0, 1, nu - 1):
            for sg in range(3):
                for a in range(rpu):
                    assert sc[pos, sg, a, :3].tolist() == d3[sg, o[pos] + a * nu, :3].tolist()
                    assert sc[pos, sg, a, 3] == o[pos]
        ident = P.schedule(desc, 64, 3, rpu, None)
        assert ident[:, 0, 0, 3].tolist() == list(range(nu))
        with pytest.raises(ValueError, match="permutation"):
            P.schedule(desc, 64, 3, rpu, np.zeros(nu, np.int32))
    u = synth.synth_matrix(16 * 8, 16 * 8, 0.25, 5)
    assert P.unit_order(u["offsets"], 8, 1).tolist() == list(range(8))             # uniform rows keep natural order


def _barrier_cost(desc, Rb, nseg, rpu, order, waves, upw):
    """Sum over workgroup windows and K segments of the heaviest wave's executed block pairs."""
    nu = Rb // rpu
    nb = desc.reshape(nseg, Rb, 4)[:, :, 2]
    pairs = (nb + 3) // 4 * 2
    cost = pairs[:, :nu] + (pairs[:, nu:] if rpu == 2 else 0)                     # [nseg, nu]
    total = 0
    for p0 in range(0, nu, waves * upw):
        win = order[p0:p0 + waves * upw]
        for s in range(nseg):
            total += max(sum(cost[s, u] for u in win[w::waves]) for w in range(waves))
    return total


@pytest.mark.parametrize("rpu,Rb,zipf", [(1, 128, 0.0), (2, 128, 0.0), (1, 72, 1.2), (2, 200, 1.2)])
def test_unit_order_segments(rpu, Rb, zipf):
    Cb, seg = 90, 31
    m = synth.synth_matrix(16 * Rb, 16 * Cb, 0.25, 6, zipf_s=zipf)
    nnz = int(m["offsets"][-1])
    dw, sdup = P.encode_blocks(O.pack_ternary_codes(m["codes"]), nnz, m["scales"])
    desc, _, _, _ = P.octet_layout(m["offsets"], Rb, Cb, seg, dw, sdup, m["col_idx"])
    nseg, nu = 3, Rb // rpu
    o = P.unit_order(m["offsets"], Rb, rpu)
    o2 = P.unit_order_segments(desc, Rb, nseg, rpu, o)
    waves, upw = P.SCHED_GROUP, P.SCHED_UNITS_PER_WAVE[rpu]
    per = waves * upw
    for p0 in range(0, nu, per):                                                    # every window keeps its units
        assert sorted(o2[p0:p0 + per].tolist()) == sorted(o[p0:p0 + per].tolist())
    before, after = _barrier_cost(desc, Rb, nseg, rpu, o, waves, upw), _barrier_cost(desc, Rb, nseg, rpu, o2, waves, upw)
    assert after <= before
    if zipf == 0.0:
        assert after < 0.97 * before                                                # uniform rows: > 3 % less waiting
    # a kernel that gives a wave half as many units runs each half of a full window as its own workgroup: the halves
    # hold the same number of executed block pairs to within a few units (the greedy alone would put a wave's heaviest
    # units all in the first half)
    pairs = (desc.reshape(nseg, Rb, 4)[:, :, 2] + 3) // 4 * 2
    ucost = (pairs[:, :nu] + (pairs[:, nu:] if rpu == 2 else 0)).sum(axis=0)
    for p0 in range(0, nu - per + 1, per):
        first, second = ucost[o2[p0:p0 + per // 2]].sum(), ucost[o2[p0 + per // 2:p0 + per]].sum()
        assert abs(int(first) - int(second)) <= 0.03 * (first + second), (p0, first, second)
    one = P.unit_order_segments(desc[:Rb * 4], Rb, 1, rpu, o)                       # a single segment: untouched
    assert np.array_equal(one, o)


def test_tile_queries():
    L = _lib.lib()
    assert L.mortar_prefill_max_seg_cb() == 155
    assert L.mortar_route_tile(128, 4096) == 32 and L.mortar_route_tile(48, 4096) == 64
    assert L.mortar_route_tile(128, 1) == 4 and L.mortar_route_tile(128, 16) == 16
    assert L.mortar_route_tile(352, 4096) == 0                                      # too wide for routed skipping
    assert L.mortar_stack_table_bytes(3) % 16 == 0 and L.mortar_stack_table_bytes(0) == 0


@pytest.mark.parametrize("rpu,kseg,mb", [(1, 1000, 1 << 20), (2, 1000, 1 << 20), (1, 7, 3), (2, 16, 4)])
def test_decode_worklist_covers_every_block_once(rpu, kseg, mb):
    m = synth.synth_matrix(16 * 12, 16 * 40, 0.3, 6, zipf_s=1.2)
    ent, nslots, row_slots = P.decode_worklist(m["offsets"], m["col_idx"], 12, 40, rpu, kseg, mb)
    assert ent.shape[0] % 4 == 0
    seen = np.zeros(m["offsets"][-1], int)
    slots = {}
    for g in range(0, len(ent), 4):
        assert len({e[7] for e in ent[g:g + 4]}) == 1                                  # one segment per workgroup
    for e in ent:
        if e[0] < 0:
            continue
        for row, p, c in ((e[0], e[1], e[2]), (e[3], e[4], e[5])):
            if row < 0:
                continue
            assert c <= mb and m["offsets"][row] <= p and p + c <= m["offsets"][row + 1]
            cols = m["col_idx"][p:p + c]
            assert ((cols >= e[7] * kseg) & (cols < (e[7] + 1) * kseg)).all()
            seen[p:p + c] += 1
        slots.setdefault(e[0], []).append(e[6])
        if rpu == 2:
            assert e[3] == e[0] + 6
    assert (seen == 1).all()
    for u, s in slots.items():
        assert sorted(s) == list(range(len(s))) and row_slots[u] == len(s)
    assert nslots == max(len(s) for s in slots.values())


def test_module_carve_matches_oracle_layout():
    torch.manual_seed(0)
    lin = mortar_amd.MortarLinear(16 * 6, 16 * 5, bias=False)
    rng = np.random.default_rng(7)
    mask = rng.random((5, 6)) < 0.5
    mask[np.arange(5), rng.integers(0, 6, 5)] = True
    w = lin._cms.weight.detach().numpy().copy()
    lin._cms.set_block_mask(torch.from_numpy(mask), 16)
    nnz = lin.carve(16)
    c = O.carve(w, mask, 16)
    assert nnz == mask.sum() and lin.is_compact
    sd = lin.state_dict()
    for k in ("mortar_data", "mortar_row_indices", "mortar_column_indices", "mortar_offsets",
              "mortar_column_indices_t", "mortar_offsets_t", "mortar_block_offsets_t"):
        assert np.array_equal(sd["_cms." + k].numpy(), c[k]), k
        assert sd["_cms." + k].numpy().dtype == c[k].dtype
    assert "_cms.mortar_ternary" in sd
    with pytest.raises(AssertionError):
        lin.carve(16)


def test_pack_mortar_ternary_and_state_dict_round_trip():
    torch.manual_seed(1)
    lin = mortar_amd.MortarLinear(64, 48, bias=False)
    info = mortar_amd.shrink_mlp_to_mortar_ternary(lin, 0.5, 16, generator=torch.Generator().manual_seed(3))
    cms = lin._cms
    assert type(cms).__name__ == "CMSBlockLinear" and cms._mortar and cms._packed_shape == (info["nnz"], 16, 16)
    assert cms.mortar_packed.dtype == torch.uint8 and cms.mortar_packed.numel() == info["nnz"] * 64
    eff = cms._mortar_effective_data().float()
    mags = eff.abs()[eff != 0].unique()
    assert len(mags) == 1 and torch.isclose(mags[0], cms.mortar_scale.to(torch.bfloat16).float())
    # oracle quantiser agrees
    lin2 = mortar_amd.MortarLinear(64, 48, bias=False)
    lin2.load_state_dict(lin.state_dict())
    assert lin2._cms._mortar and torch.equal(lin2._cms.mortar_packed, cms.mortar_packed)
    assert lin2._cms._packed_shape == cms._packed_shape
    # per-block variant
    lin3 = mortar_amd.MortarLinear(64, 48, bias=False)
    mortar_amd.shrink_mlp_to_mortar_ternary(lin3, 0.5, 16, per_block=True)
    assert lin3._cms.mortar_scale.shape == (lin3._cms._packed_shape[0],)


def test_quantize_mirror_matches_oracle():
    from mortar_amd.deploy_quant import _ternary_quantize, _ternary_quantize_per_block
    w = torch.randn(7, 16, 16, generator=torch.Generator().manual_seed(2))
    q, s = _ternary_quantize(w)
    qo, so = O.ternary_quantize(w.numpy())
    assert np.array_equal(q.numpy(), qo) and np.isclose(float(s), so, rtol=1e-6)
    q, s = _ternary_quantize_per_block(w)
    qo, so = O.ternary_quantize_per_block(w.numpy())
    assert np.array_equal(q.numpy(), qo) and np.allclose(s.numpy(), so, rtol=1e-6)
    assert np.array_equal(mortar_amd.pack_ternary_codes(q).numpy(), O.pack_ternary_codes(qo))
    assert np.array_equal(synth.flat_pack(qo), O.pack_ternary_codes(qo))


def test_product_fails_loudly_without_gpu_or_library(monkeypatch):
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    m = synth.synth_matrix(32, 64, 0.5, 0)
    W = synth.to_pack(m, "cpu")
    with pytest.raises(RuntimeError, match="no CPU path"):
        mortar_amd.ops.spmm(x, W)
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmortar_hip.so")
    with pytest.raises(RuntimeError, match="has not been built"):
        _lib.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "morph-orchestrates-recursive-pruned-hierarchies_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                assert "oracle" not in open(os.path.join(dirpath, f)).read().lower(), f


def test_synth_generators_are_deterministic_and_shaped():
    a, b = synth.synth_matrix(2048, 768, 0.25, 1), synth.synth_matrix(2048, 768, 0.25, 1)
    assert all(np.array_equal(a[k], b[k]) for k in ("codes", "scales", "col_idx", "offsets"))
    assert a["offsets"][-1] == 1536 and (np.diff(a["offsets"]) == 12).all()
    frac = [(a["codes"] == v).mean() for v in (-1, 0, 1)]
    assert np.allclose(frac, [0.3, 0.4, 0.3], atol=0.01)
    z = synth.synth_matrix(16 * 128, 16 * 352, 0.25, 2, zipf_s=1.2)
    cnt = np.diff(z["offsets"])
    assert cnt.min() >= round(0.05 * 352) and cnt.max() <= round(0.60 * 352)
    assert abs(cnt.mean() / 352 - 0.25) < 0.02 and cnt.std() > 10


def test_bench_refuses_more_than_one_gpu():
    import subprocess, sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)


def test_octet_positions_match_the_octet_layout():
    """pos[j] must be where mortar_octet_layout_host put block j, for one and for several K segments."""
    from mortar_amd import pack, synth
    for shape, seg in (((16 * 9, 16 * 40), 40), ((16 * 7, 16 * 50), 17), ((16 * 5, 16 * 352), 118)):
        m = synth.synth_matrix(shape[0], shape[1], 0.3, seed=3, zipf_s=1.2)
        Rb, Cb = shape[0] // 16, shape[1] // 16
        nnz = m["col_idx"].size
        codes = (np.arange(nnz * 16, dtype=np.uint64) * 2654435761 % (1 << 32)).astype(np.uint32)
        sdup = np.arange(1, nnz + 1, dtype=np.uint32)
        grp, codes_o, sd_o, col_o = pack.octet_layout(m["offsets"], Rb, Cb, seg, codes, sdup, m["col_idx"])
        pos = pack.octet_positions(m["offsets"], Rb, Cb, seg, m["col_idx"])
        assert len(set(pos.tolist())) == nnz and pos.max() < sd_o.size
        assert np.array_equal(sd_o[pos], sdup)
        co = codes_o.reshape(-1, 16, 4)
        for j in range(0, nnz, 7):
            assert np.array_equal(co[pos[j] >> 2, :, pos[j] & 3], codes[j * 16:(j + 1) * 16])


def test_transpose_topology_against_the_oracle():
    """The W^T topology equals the oracle's restatement of stk's _transpose (stable order inside a column)."""
    from mortar_amd import pack, synth
    m = synth.synth_matrix(16 * 12, 16 * 30, 0.2, seed=5, zipf_s=1.2)
    off_t, col_t, src = pack.transpose_topology(m["offsets"], m["col_idx"], 12, 30)
    ct, ot, bt = O.transpose_meta((16 * 12, 16 * 30), 16, m["row_idx"], m["col_idx"])
    assert np.array_equal(off_t, ot) and np.array_equal(col_t, ct) and np.array_equal(src, bt)
    with pytest.raises(ValueError):
        pack.transpose_topology(m["offsets"], m["col_idx"][::-1].copy(), 12, 30)


def test_sdd_plan_partitions_the_blocks():
    """Every kept block appears exactly once, inside its workgroup's row window and K segment."""
    from mortar_amd import synth
    L = _lib.lib()
    for shape, nbw in (((16 * 40, 16 * 30), 22), ((16 * 9, 16 * 352), 8), ((16 * 704, 16 * 128), 22), ((16 * 704, 16 * 128), 12)):
        m = synth.synth_matrix(shape[0], shape[1], 0.25, seed=9, zipf_s=1.2)
        Rb, Cb = shape[0] // 16, shape[1] // 16
        off, col = np.ascontiguousarray(m["offsets"], np.int32), np.ascontiguousarray(m["col_idx"], np.int16)
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        n = L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, nbw, None, 0)
        plan = np.empty(n, np.int32)
        assert L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, nbw, vp(plan), n) == n
        assert L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, nbw, vp(plan), n - 1) < 0
        assert L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, 9, None, 0) < 0        # not a built group size
        n_wg, seg_cb, nseg, tab = plan[0], plan[1], plan[2], plan[3]
        assert tab + n_wg == n
        G = (tab - 4 - 4 * n_wg) // (2 * n_wg)
        assert G == 16 * nbw
        desc = plan[4:4 + 4 * n_wg].reshape(n_wg, 4)
        ej = plan[4 + 4 * n_wg:4 + 4 * n_wg + n_wg * G].reshape(n_wg, G)
        eo = plan[4 + 4 * n_wg + n_wg * G:tab].reshape(n_wg, G)
        # workgroups are stored segment by segment; the launch order lists every workgroup once, by its position
        # inside the segment first (row groups of about the same rows side by side), then by segment
        assert (np.diff(desc[:, 2]) >= 0).all()
        order = plan[tab:]
        assert sorted(order.tolist()) == list(range(n_wg))
        first = np.searchsorted(desc[:, 2], np.arange(nseg))
        key = [(w - first[desc[w, 2]], desc[w, 2]) for w in order]
        assert key == sorted(key)
        assert nseg >= -(-Cb // seg_cb) and seg_cb <= 44 and seg_cb % 4 == 0
        seen = ej[ej >= 0]
        assert sorted(seen.tolist()) == list(range(col.size))
        assert (eo >= 0).all()                                  # empty slots repeat a valid tile
        row_of = np.repeat(np.arange(Rb), np.diff(off))
        for w in range(n_wg):
            row0, nrows, seg, nb = desc[w]
            js = ej[w][ej[w] >= 0]
            assert nb == js.size and 1 <= nrows <= 32
            assert np.array_equal(eo[w][ej[w] >= 0] >> 20, row_of[js] - row0) and (row_of[js] - row0 < nrows).all()
            off = eo[w] & 0xfffff                               # LDS offset of the block's column: quad * 4224 + (col & 3) * 32
            tile = (off // 4224) * 4 + (off % 4224) // 32
            assert ((off % 4224) % 32 == 0).all() and (off % 4224 < 128).all() and (tile < seg_cb).all() and ((eo[w] >> 20) < nrows).all()
            assert np.array_equal(tile[ej[w] >= 0], col[js] - seg * seg_cb) and (col[js] // seg_cb == seg).all()


def test_sdd_blocks_per_wave_is_a_built_size_and_fills_the_chip():
    """The chosen group size is one of the built kernels; at the headline shapes and 4096 tokens its plan has a count
    of token ranges that puts 200 to 256 workgroups on the 256 CUs (one per CU, one round)."""
    from mortar_amd import synth
    L = _lib.lib()
    vp = lambda a: a.ctypes.data_as(C.c_void_p)
    for shape, M in (((11264, 2048), 4096), ((2048, 5632), 4096), ((64, 96), 7), ((11264, 2048), 0), ((2048, 5632), 16384)):
        m = synth.synth_matrix(shape[0], shape[1], 0.25, seed=3)
        Rb, Cb = shape[0] // 16, shape[1] // 16
        off, col = np.ascontiguousarray(m["offsets"], np.int32), np.ascontiguousarray(m["col_idx"], np.int16)
        nbw = L.mortar_sdd_blocks_per_wave_host(vp(off), vp(col), Rb, Cb, M)
        assert nbw in (8, 10, 12, 14, 16, 18, 20, 22)
        n = L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, nbw, None, 0)
        plan = np.empty(n, np.int32)
        assert L.mortar_sdd_plan_host(vp(off), vp(col), Rb, Cb, nbw, vp(plan), n) == n
        ws = L.mortar_sdd_workspace_bytes(int(plan[0]), col.size, nbw, M)
        ranges = ws // (col.size * 1024)
        assert ws == ranges * col.size * 1024 and 1 <= ranges <= 16
        if M >= 4096:
            assert 200 <= ranges * plan[0] <= 256, (shape, M, nbw, ranges, plan[0])
    assert L.mortar_sdd_blocks_per_wave_host(vp(off), vp(col), Rb, Cb, -1) < 0
    assert L.mortar_sdd_workspace_bytes(4, 16, 9, 64) < 0


def test_operator_fake_implementations_trace_without_a_gpu():
    """stk_dds / stk_sdd_at_b carry fake (meta) implementations, as the reference's custom ops do
    (custom_ops.py:59-65, 93-96): shapes and dtypes propagate under FakeTensorMode with no device present."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        lhs = torch.empty(40, 96, dtype=torch.bfloat16, device="cuda")
        data = torch.empty(10, 16, 16, dtype=torch.bfloat16, device="cuda")
        off = torch.empty(9, dtype=torch.int32, device="cuda")
        idx = torch.empty(10, dtype=torch.int16, device="cuda")
        y = mortar_amd.stk_dds(lhs, data, off, idx, idx, off, idx, off, 96, 128, True)
        assert tuple(y.shape) == (40, 128) and y.dtype == torch.bfloat16
        dx = mortar_amd.stk_dds(y, data, off, idx, idx, off, idx, off, 128, 96, False)
        assert tuple(dx.shape) == (40, 96)
        dw = mortar_amd.stk_sdd_at_b(y, lhs, data, off, idx, idx)
        assert tuple(dw.shape) == (10, 16, 16) and dw.dtype == torch.bfloat16


def test_module_carve_at_coarser_blocking_matches_oracle_layout():
    """carve(blocking=64) with a 16-tile prune mask: a block is kept when any tile inside it is, pruned tiles inside
    kept blocks hold zeros (reference block_sparse.py:859-890); same arrays as the oracle's carve at that blocking."""
    torch.manual_seed(4)
    lin = mortar_amd.MortarLinear(64 * 3, 64 * 2, bias=False)
    rng = np.random.default_rng(8)
    tiles = rng.random((8, 12)) < 0.15
    tiles[0, 0] = tiles[4, 5] = True                                     # every 64-row keeps something
    w = lin._cms.weight.detach().numpy().copy()
    lin._cms._prune_mask = torch.from_numpy(tiles)
    lin.carve(64)
    bm = tiles.reshape(2, 4, 3, 4).any(axis=(1, 3))
    c = O.carve(w * np.kron(tiles, np.ones((16, 16), np.float32)), bm, 64)
    sd = lin.state_dict()
    for k in ("mortar_data", "mortar_row_indices", "mortar_column_indices", "mortar_offsets"):
        assert np.array_equal(sd["_cms." + k].numpy(), c[k]), k


@pytest.mark.parametrize("B,per_block", [(128, False), (64, True), (32, False)])
def test_recut_blocks_is_the_same_matrix(B, per_block):
    """A BCSR carved at blocking B re-cut into 16 x 16 blocks scatters to the same dense matrix (oracle to_dense of both
    layouts), keeps row-major order with ascending columns, drops exactly the all-zero sub-blocks and hands every
    sub-block its block's scale."""
    rng = np.random.default_rng(B)
    Rb, Cb = 3, 4
    mask = rng.random((Rb, Cb)) < 0.6
    mask[np.arange(Rb), rng.integers(0, Cb, Rb)] = True
    r, c = np.nonzero(mask)
    nnz = r.size
    codes = rng.integers(-1, 2, (nnz, B, B)).astype(np.int8)
    zero_tiles = rng.random((nnz, B // 16, B // 16)) < 0.4               # pruned 16-tiles inside kept blocks
    codes *= ~np.kron(zero_tiles, np.ones((16, 16), bool))
    scales = rng.uniform(0.01, 0.1, nnz).astype(np.float32) if per_block else np.float32(0.037)
    c16, s16, col16, off16 = P.recut_blocks(codes, scales, r, c, Rb * B)
    assert c16.shape[0] == int((~zero_tiles).sum()) - int((codes.reshape(nnz, B // 16, 16, B // 16, 16).transpose(0, 1, 3, 2, 4)
                                                           .reshape(nnz, B // 16, B // 16, -1).any(-1) != ~zero_tiles).sum())
    assert off16[0] == 0 and off16[-1] == c16.shape[0] and off16.size == Rb * B // 16 + 1
    row16 = np.repeat(np.arange(Rb * B // 16), np.diff(off16))
    for rr in range(Rb * B // 16):
        cols = col16[off16[rr]:off16[rr + 1]]
        assert (np.diff(cols.astype(int)) > 0).all()
    sc = np.broadcast_to(np.asarray(scales, np.float32).reshape(-1), (nnz,))
    big = O.to_dense(codes.astype(np.float32) * sc[:, None, None], r, c, (Rb * B, Cb * B), B)
    s16b = np.broadcast_to(np.asarray(s16, np.float32).reshape(-1), (c16.shape[0],))
    small = O.to_dense(c16.astype(np.float32) * s16b[:, None, None], row16, col16, (Rb * B, Cb * B), 16)
    assert np.array_equal(big, small)
    assert c16.reshape(c16.shape[0], -1).any(axis=1).all()               # no all-zero block kept
    with pytest.raises(ValueError):
        P.recut_blocks(np.zeros((1, 24, 24), np.int8), 1.0, [0], [0], 24)


def test_layer_carved_at_128_loads_and_packs_on_the_host():
    """The reference's checkpoints are carved at blocking 128: such a state dict loads, and mortar_pack() re-cuts it
    into a 16 x 16 pack whose decoded blocks scatter to the layer's effective dense weight."""
    torch.manual_seed(5)
    src = mortar_amd.MortarLinear(256, 384, bias=False)
    info = mortar_amd.shrink_mlp_to_mortar_ternary(src, 0.5, 128, generator=torch.Generator().manual_seed(6))
    assert src._cms._mortar_blocking == 128 and src._cms._packed_shape[1:] == (128, 128)
    dst = mortar_amd.MortarLinear(256, 384, bias=False)
    dst.load_state_dict(src.state_dict())
    cms = dst._cms
    assert cms._mortar_blocking == 128 and cms._packed_shape == src._cms._packed_shape
    W = cms.mortar_pack()
    assert W is cms.mortar_pack() and W.Rb == 24 and W.Cb == 16
    eff = cms._mortar_effective_data().float().numpy()
    dense = O.to_dense(eff, cms.mortar_row_indices.numpy(), cms.mortar_column_indices.numpy(), (384, 256), 128)
    q16 = P.decode_blocks(W.codes.numpy().view(np.uint32))
    s = float(O.bf16_round(np.array([float(cms.mortar_scale)], np.float32))[0])
    row16 = np.repeat(np.arange(W.Rb), np.diff(W.h_offsets))
    got = O.to_dense(q16.astype(np.float32) * s, row16, W.h_col, (384, 256), 16)
    assert np.array_equal(got, dense)
