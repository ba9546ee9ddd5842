"""Seeded random sweeps of the GPU entry points against the oracle: shapes, densities, row counts, K segment widths,
scale modes and gating drawn at random (fixed seeds), so that combinations no hand-written case names are exercised.
Each failing case prints its configuration.  The bars are those of test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from mortar_amd import ops, synth
from mortar_amd.pack import MortarPack, decode_blocks
from oracle import mortar_oracle as O
from util import assert_close_bf16, oracle_spmm, to_dev, to_np

pytestmark = pytest.mark.gpu


def _pack(m, dev, **kw):
    return MortarPack(synth.flat_pack(m["codes"]), m["scales"], m["col_idx"], m["offsets"], m["shape"][0], m["shape"][1], dev, **kw)


@pytest.mark.parametrize("seed", [101, 102])
def test_random_mlp_shapes_prefill_and_decode_tiles(dev, seed):
    """gate_up + SwiGLU, down, plain gate_up product, gated and list-routed gate_up, masked down."""
    rng = np.random.default_rng(seed)
    for it in range(40):
        dm_b = int(rng.choice([1, 2, 3, 5, 8, 16, 30, 48, 77, 78, 128, 155, 156, 200]))
        dff_b = int(rng.choice([1, 2, 4, 7, 16, 22, 40, 64, 130, 352]))
        if dm_b * dff_b > 352 * 48:
            dff_b = 22
        cfg = dict(it=it, d_model=dm_b * 16, d_ff=dff_b * 16, dens=float(rng.choice([0.05, 0.1, 0.25, 0.5, 1.0])),
                   zipf=None if rng.random() < 0.5 else 1.2,
                   M=int(rng.choice([1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 96, 127, 129, 200, 257])),
                   seg=None if rng.random() < 0.6 else int(rng.integers(1, 80)), uniform=bool(rng.random() < 0.25),
                   stream4=bool(rng.random() < 0.7), seed=int(rng.integers(1, 10000)))
        what = f"seed {seed} case {cfg}"
        spec = synth.synth_mlp(cfg["d_model"], cfg["d_ff"], cfg["dens"], seed=cfg["seed"], zipf_s=cfg["zipf"])
        if cfg["uniform"]:
            spec["gate_up"]["scales"], spec["down"]["scales"] = np.float32(0.05), np.float32(0.03)
        M = cfg["M"]
        x = synth.synth_x(M, cfg["d_model"], cfg["seed"] + 1)
        xd = to_dev(x, dev)
        Wgu = _pack(spec["gate_up"], dev, seg_cb=cfg["seg"], prefill_stream=cfg["stream4"])
        Wdn = _pack(spec["down"], dev, seg_cb=cfg["seg"], prefill_stream=cfg["stream4"])
        ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
        h = ops.gateup_swiglu(xd, Wgu)
        assert_close_bf16(to_np(h), ref["h"], what + " h", ulps=8)
        assert_close_bf16(to_np(ops.spmm(h, Wdn)), oracle_spmm(to_np(h), spec["down"]), what + " y", ulps=8)
        assert_close_bf16(to_np(ops.spmm(xd, Wgu)), oracle_spmm(x, spec["gate_up"]), what + " gu", ulps=8)
        ncl, k = dff_b, max(1, dff_b // 3)
        logits = synth.synth_logits(M, ncl, cfg["seed"] + 2)
        g_ref, act_ref = O.remoe_gates(logits, k)
        gates, active = ops.remoe_gates(torch.from_numpy(logits).to(dev), k)
        assert np.array_equal(active.cpu().numpy().astype(bool), act_ref), what
        refg = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
        hg = ops.gateup_swiglu(xd, Wgu, gates=gates)
        assert_close_bf16(to_np(hg), refg["h"], what + " h gated", ulps=8)
        tile = ops.route_tile(Wgu, M)
        if tile:
            hs = torch.full_like(hg, float("nan"))
            ops.gateup_swiglu(xd, Wgu, gates=gates, route=ops.remoe_route(active, tile), out=hs)
            on = np.repeat(act_ref, 16, axis=1)
            a, b = to_np(hs), to_np(hg)
            assert np.array_equal(a[on], b[on]) and np.isnan(a[~on]).all(), what + " routed tiles"
            ym = ops.spmm(hs, Wdn, active=active)
        else:
            ym = ops.spmm(hg, Wdn, active=active)
        assert_close_bf16(to_np(ym), refg["y"], what + " y routed", ulps=16)


@pytest.mark.parametrize("seed", [201, 202])
def test_random_decode_entry_points(dev, seed):
    """Small-tile launches, the work-list GEMV with gather flags and partial slots (bf16 and fp32 arithmetic), layer stacks."""
    rng = np.random.default_rng(seed)
    for it in range(60):
        dm_b = int(rng.choice([1, 2, 3, 8, 16, 32, 48, 77, 128, 160, 200]))
        ncl, cs_b = int(rng.choice([1, 2, 4, 8, 11, 22])), int(rng.choice([1, 1, 2, 4]))
        dff_b = ncl * cs_b
        cfg = dict(it=it, d_model=dm_b * 16, d_ff=dff_b * 16, ncl=ncl, dens=float(rng.choice([0.05, 0.1, 0.25, 0.5, 1.0])),
                   zipf=None if rng.random() < 0.5 else 1.2, B=int(rng.choice([1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 32, 33, 48, 64])),
                   mb=None if rng.random() < 0.5 else int(rng.integers(1, 12)), uniform=bool(rng.random() < 0.25),
                   seed=int(rng.integers(1, 10000)), n_layers=int(rng.choice([1, 2, 7])))
        what = f"seed {seed} case {cfg}"
        B, mb = cfg["B"], cfg["mb"]
        spec = synth.synth_mlp(cfg["d_model"], cfg["d_ff"], cfg["dens"], seed=cfg["seed"], zipf_s=cfg["zipf"])
        if cfg["uniform"]:
            spec["gate_up"]["scales"], spec["down"]["scales"] = np.float32(0.05), np.float32(0.03)
        x = synth.synth_x(B, cfg["d_model"], cfg["seed"] + 1)
        xd = to_dev(x, dev)
        Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
        g_ref, _ = O.remoe_gates(synth.synth_logits(B, ncl, cfg["seed"] + 2), max(1, ncl // 3))
        gates = torch.from_numpy(g_ref).to(dev)
        ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
        refg = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
        h = ops.gemv(xd, Wgu, swiglu_out=True)
        assert_close_bf16(to_np(h), ref["h"], what + " h", ulps=8)
        assert_close_bf16(to_np(ops.gemv(h, Wdn)), oracle_spmm(to_np(h), spec["down"]), what + " y", ulps=8)
        ract, cact = ops.route_flags(gates, cfg["d_ff"])
        hg = ops.gemv(xd, Wgu, swiglu_out=True, gates=gates, row_act=ract, max_blocks=mb)
        assert_close_bf16(to_np(hg), refg["h"], what + " h flagged", ulps=8)
        assert_close_bf16(to_np(ops.gemv(hg, Wdn, col_act=cact, max_blocks=mb)), refg["y"], what + " y flagged", ulps=16)
        assert_close_bf16(to_np(ops.gemv(xd, Wgu, swiglu_out=True, max_blocks=mb if mb else 5)), ref["h"], what + " h partial", ulps=8)
        gm = spec["gate_up"]
        sc = np.broadcast_to(gm["scales"], (int(gm["offsets"][-1]),)) if cfg["uniform"] else gm["scales"]
        gu64 = O.mortar_gemv(x, gm["codes"], sc, gm["col_idx"], gm["offsets"]).astype(np.float64)
        got = ops.gemv_f32(torch.from_numpy(x).to(dev), Wgu, max_blocks=mb).cpu().numpy()
        assert np.abs(got - gu64).max() <= 3e-6 * max(np.abs(gu64).max(), 1e-30), what + " gemv_f32"
        if B <= 16:
            n = cfg["n_layers"]
            hs = [torch.empty((B, cfg["d_ff"]), dtype=torch.bfloat16, device=dev) for _ in range(n)]
            ys = [torch.empty((B, cfg["d_model"]), dtype=torch.bfloat16, device=dev) for _ in range(n)]
            ops.LayerStack([Wgu] * n, [xd] * n, hs, swiglu=True).run()
            ops.LayerStack([Wdn] * n, hs, ys, swiglu=False).run()
            assert_close_bf16(to_np(hs[-1]), ref["h"], what + " stack h", ulps=8)
            assert_close_bf16(to_np(ys[-1]), oracle_spmm(to_np(hs[-1]), spec["down"]), what + " stack y", ulps=8)


@pytest.mark.parametrize("seed", [301])
def test_random_backward_products(dev, seed):
    """dW on the topology and dX through the transposed pack after a device re-pack."""
    rng = np.random.default_rng(seed)
    for it in range(60):
        Rb = int(rng.choice([1, 2, 3, 7, 16, 31, 32, 33, 40, 64, 70, 128]))
        Cb = int(rng.choice([1, 2, 5, 16, 43, 44, 45, 48, 88, 89, 128, 200, 352]))
        if Rb * Cb > 128 * 128:
            Rb = 16
        cfg = dict(it=it, Rb=Rb, Cb=Cb, dens=float(rng.choice([0.03, 0.1, 0.25, 0.5, 1.0])), zipf=None if rng.random() < 0.5 else 1.2,
                   M=int(rng.choice([1, 2, 15, 16, 17, 31, 33, 64, 100, 255, 256, 257, 511, 700])), per_block=bool(rng.random() < 0.5),
                   seed=int(rng.integers(1, 10000)))
        what = f"seed {seed} case {cfg}"
        M = cfg["M"]
        m = synth.synth_matrix(Rb * 16, Cb * 16, cfg["dens"], seed=cfg["seed"], zipf_s=cfg["zipf"])
        a, b = synth.synth_x(M, Rb * 16, seed=cfg["seed"] + 1), synth.synth_x(M, Cb * 16, seed=cfg["seed"] + 2)
        ref_dw = O.sdd_at_b(O.bf16_round(a), O.bf16_round(b), m["row_idx"], m["col_idx"])
        Wd = synth.to_pack(m, dev)
        assert_close_bf16(to_np(ops.sdd(to_dev(a, dev), to_dev(b, dev), Wd)), ref_dw, what + " dW")
        nbw = int(np.random.default_rng(cfg["seed"] + 9).choice([8, 10, 12, 14, 16, 18, 20, 22]))      # any built group size
        assert_close_bf16(to_np(ops.sdd(to_dev(a, dev), to_dev(b, dev), Wd, blocks_per_wave=nbw)), ref_dw, what + f" dW group size {nbw}")
        nnz = m["col_idx"].size
        g = np.random.Generator(np.random.PCG64(cfg["seed"] + 3))
        v = g.standard_normal((nnz, 16, 16), dtype=np.float32) * g.uniform(0.01, 0.1, (nnz, 1, 1)).astype(np.float32)
        vt = torch.from_numpy(v).to(torch.bfloat16).to(dev)
        W = MortarPack(None, None, m["col_idx"], m["offsets"], Rb * 16, Cb * 16, dev)
        s = W.requantize(vt, per_block=cfg["per_block"]).cpu().numpy()
        Wt = W.transposed()
        Wt.requantize(vt, per_block=cfg["per_block"], transpose=True)
        cw = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
        dense = O.to_dense(cw.astype(np.float32) * O.bf16_round(np.broadcast_to(s, (nnz,)))[:, None, None], m["row_idx"], m["col_idx"],
                           (Rb * 16, Cb * 16)).astype(np.float64)
        assert_close_bf16(to_np(ops.spmm(to_dev(a, dev), Wt)), (O.bf16_round(a).astype(np.float64) @ dense).astype(np.float32),
                          what + " dX", ulps=8)
        assert_close_bf16(to_np(ops.spmm(to_dev(b, dev), W)), (O.bf16_round(b).astype(np.float64) @ dense.T).astype(np.float32),
                          what + " y", ulps=8)


@pytest.mark.parametrize("seed", [401])
def test_random_fp32_decode_products(dev, seed):
    """mortar_gemv in fp32 arithmetic on random shapes with one scale per matrix (the SpMM-kernel form: 3 * B term rows
    through 4-, 8-, 16-token and prefill tiles, one or several K segments, with and without the 4-bit stream) and with a
    scale per block (the work-list kernel), against the oracle's float64 sums."""
    rng = np.random.default_rng(seed)
    for it in range(40):
        Rb = int(rng.choice([1, 2, 7, 16, 33, 64, 128, 200]))
        Cb = int(rng.choice([1, 2, 5, 16, 48, 96, 128, 155, 156, 352]))
        cfg = dict(it=it, Rb=Rb, Cb=Cb, dens=float(rng.choice([0.1, 0.25, 0.5, 1.0])), zipf=None if rng.random() < 0.5 else 1.2,
                   B=int(rng.choice([1, 2, 4, 5, 6, 16, 21, 22, 43, 64])), one=bool(rng.random() < 0.7),
                   seg=None if rng.random() < 0.6 else int(rng.integers(1, 80)), stream4=bool(rng.random() < 0.6),
                   seed=int(rng.integers(1, 10000)))
        what = f"seed {seed} case {cfg}"
        m = synth.synth_matrix(Rb * 16, Cb * 16, cfg["dens"], seed=cfg["seed"], zipf_s=cfg["zipf"])
        if cfg["one"]:
            m["scales"] = m["scales"][:1] * np.float32(1.2345)
        W = _pack(m, dev, seg_cb=cfg["seg"], prefill_stream=cfg["stream4"])
        x = (np.random.default_rng(cfg["seed"] + 1).standard_normal((cfg["B"], Cb * 16)) * 1.37).astype(np.float32)
        ref = O.mortar_gemv(x, m["codes"], m["scales"], m["col_idx"], m["offsets"]).astype(np.float64)
        got = ops.gemv_f32(torch.from_numpy(x).to(dev), W).cpu().numpy()
        assert np.abs(got - ref).max() <= 3e-6 * max(np.abs(ref).max(), 1e-30), what


@pytest.mark.parametrize("seed", [501])
def test_random_wide_k_shapes(dev, seed):
    """Rows of 2048 to 21824 values (d_model / d_ff of larger models) at 1 to 300 rows: the narrow tiles of all K (2, 4,
    8 tokens, one or several per launch, 4 or 8 units per workgroup, parts shared unevenly), K-segmented 16-token tiles,
    the prefill tiles, and layer-batched launches; plain, masked and gate_up + SwiGLU with gates."""
    rng = np.random.default_rng(seed)
    for it in range(60):
        Cb = int(rng.choice([128, 192, 256, 300, 305, 320, 400, 512, 609, 610, 688, 864, 1024, 1244, 1245, 1364]))
        units = int(rng.choice([4, 8, 24, 64, 128, 256, 352, 700, 1364]))
        dens = float(rng.choice([0.03, 0.06, 0.125, 0.25]))
        if units * Cb * dens > 40000:
            dens = 40000 / (units * Cb)
        cfg = dict(it=it, Cb=Cb, units=units, dens=round(dens, 4), zipf=None if rng.random() < 0.5 else 1.2,
                   M=int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 48, 63, 64, 65, 100, 128, 129, 200, 256, 257, 300])),
                   uniform=bool(rng.random() < 0.3), stream4=bool(rng.random() < 0.6), kind=int(rng.choice([0, 1, 3])),
                   stack=bool(rng.random() < 0.5), seed=int(rng.integers(1, 10000)))
        what = f"seed {seed} case {cfg}"
        M = cfg["M"]
        if cfg["kind"] == 1:
            spec = synth.synth_mlp(Cb * 16, units * 16, dens, seed=cfg["seed"], zipf_s=cfg["zipf"])
            m = spec["gate_up"]
        else:
            m = synth.synth_matrix(units * 16, Cb * 16, dens, seed=cfg["seed"], zipf_s=cfg["zipf"])
        if cfg["uniform"]:
            m["scales"] = np.float32(0.04)
        W = _pack(m, dev, prefill_stream=cfg["stream4"])
        x = synth.synth_x(M, Cb * 16, cfg["seed"] + 1)
        xd = to_dev(x, dev)
        if cfg["kind"] == 0:
            ref = oracle_spmm(x, m)
            assert_close_bf16(to_np(ops.spmm(xd, W)), ref, what + " spmm", ulps=8)
            if M <= 64:
                assert_close_bf16(to_np(ops.gemv(xd, W)), ref, what + " gemv", ulps=8)
                if cfg["stack"]:
                    ys = [torch.full((M, units * 16), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(2)]
                    ops.LayerStack([W, W], [xd, xd], ys, swiglu=False).run()
                    assert_close_bf16(to_np(ys[1]), ref, what + " stack", ulps=8)
        elif cfg["kind"] == 3:
            act = O.remoe_gates(synth.synth_logits(M, Cb, cfg["seed"] + 2), max(1, Cb // 4))[1]
            got = ops.spmm(xd, W, active=torch.from_numpy(act.astype(np.uint8)).to(dev))
            assert_close_bf16(to_np(got), oracle_spmm(x * np.repeat(act, 16, axis=1), m), what + " masked", ulps=8)
        else:
            g_ref = O.remoe_gates(synth.synth_logits(M, units, cfg["seed"] + 2), max(1, units // 3))[0]
            ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
            refg = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
            assert_close_bf16(to_np(ops.gateup_swiglu(xd, W)), ref["h"], what + " h", ulps=8)
            assert_close_bf16(to_np(ops.gateup_swiglu(xd, W, gates=torch.from_numpy(g_ref).to(dev))), refg["h"], what + " gated", ulps=8)
            if M <= 64 and cfg["stack"]:
                hs = [torch.full((M, units * 16), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(2)]
                ops.LayerStack([W, W], [xd, xd], hs, swiglu=True).run()
                assert_close_bf16(to_np(hs[1]), ref["h"], what + " stack h", ulps=8)


@pytest.mark.parametrize("seed", [601, 602])
def test_random_one_call_mlp_and_values_product(dev, seed):
    """The MLP as one call (tile-ordered hidden activations from 513 rows, row-major below) against the two separate calls
    (bit-equal) and the oracle on sampled rows, with gates and the fused RMSNorm drawn at random; and the product over
    stored bf16 block values (any values, ragged and empty rows, one or several K segments) against a dense float64
    product of the scattered matrix."""
    from mortar_amd.pack import BcsrTopology
    rng = np.random.default_rng(seed)
    for it in range(14):
        dm_b = int(rng.choice([2, 5, 16, 30, 48, 78, 128]))
        dff_b = int(rng.choice([4, 7, 22, 40, 130, 352]))
        cfg = dict(it=it, d_model=dm_b * 16, d_ff=dff_b * 16, dens=float(rng.choice([0.1, 0.25, 0.5])),
                   zipf=None if rng.random() < 0.5 else 1.2, M=int(rng.choice([1, 33, 200, 512, 513, 544, 777, 1025, 1500])),
                   seg=None if rng.random() < 0.6 else int(rng.integers(8, 80)), stream4=bool(rng.random() < 0.8),
                   gated=bool(rng.random() < 0.5), norm=bool(rng.random() < 0.5), seed=int(rng.integers(1, 10000)))
        what = f"seed {seed} case {cfg}"
        spec = synth.synth_mlp(cfg["d_model"], cfg["d_ff"], cfg["dens"], seed=cfg["seed"], zipf_s=cfg["zipf"])
        M = cfg["M"]
        x = synth.synth_x(M, cfg["d_model"], cfg["seed"] + 1)
        xd = to_dev(x, dev)
        Wgu = _pack(spec["gate_up"], dev, seg_cb=cfg["seg"], prefill_stream=cfg["stream4"])
        Wdn = _pack(spec["down"], dev, seg_cb=cfg["seg"], prefill_stream=cfg["stream4"])
        gates = g_ref = None
        if cfg["gated"]:
            logits = synth.synth_logits(M, dff_b, cfg["seed"] + 2)
            g_ref, _ = O.remoe_gates(logits, max(1, dff_b // 3))
            gates, _ = ops.remoe_gates(torch.from_numpy(logits).to(dev), max(1, dff_b // 3))
        nm = None
        if cfg["norm"] and ops.norm_fusable(Wgu):
            nw = O.bf16_round(1 + 0.1 * rng.standard_normal(cfg["d_model"]).astype(np.float32))
            nm = (torch.from_numpy(nw).to(torch.bfloat16).to(dev), 1e-6)
        want = ops.spmm(ops.gateup_swiglu(xd, Wgu, gates=gates, norm=nm), Wdn)
        got = ops.mlp(xd, Wgu, Wdn, gates=gates, norm=nm)
        assert torch.equal(got, want), what + " one call vs two"
        rows = rng.choice(M, min(M, 12), replace=False)
        xin = x[rows] if nm is None else O.rmsnorm(x[rows], nw, 1e-6)
        ref = O.swiglu_mlp(xin, spec["gate_up"], spec["down"], gates=None if g_ref is None else g_ref[rows])
        assert_close_bf16(to_np(got)[rows], ref["y"], what + " one call vs oracle", ulps=16)

        # any block values on the same topologies (rows emptied at random)
        for name in ("gate_up", "down"):
            m = spec[name]
            off = np.asarray(m["offsets"]).astype(np.int64)
            col = np.asarray(m["col_idx"]).astype(np.int64)
            keep = np.ones(off[-1], dtype=bool)
            for r in rng.choice(off.size - 1, max(1, (off.size - 1) // 7), replace=False):
                keep[off[r]:off[r + 1]] = False
            nb = np.array([keep[off[r]:off[r + 1]].sum() for r in range(off.size - 1)])
            off2 = np.concatenate([[0], np.cumsum(nb)]).astype(np.int32)
            col2 = col[keep].astype(np.int16)
            if off2[-1] == 0:
                continue
            vals = O.bf16_round(rng.standard_normal((int(off2[-1]), 16, 16)).astype(np.float32))
            T = BcsrTopology(off2, col2, m["shape"][0], m["shape"][1], dev)
            dense = np.zeros(m["shape"], dtype=np.float64)
            for r in range(off2.size - 1):
                for j in range(off2[r], off2[r + 1]):
                    dense[r * 16:(r + 1) * 16, col2[j] * 16:(col2[j] + 1) * 16] = vals[j]
            xv = synth.synth_x(M, m["shape"][1], cfg["seed"] + 3)
            y = ops.dds_values(to_dev(xv, dev), torch.from_numpy(vals).to(torch.bfloat16).to(dev), T)
            assert_close_bf16(to_np(y), (O.bf16_round(xv).astype(np.float64) @ dense.T).astype(np.float32), what + f" values {name}", ulps=8)
