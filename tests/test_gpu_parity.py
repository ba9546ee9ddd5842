"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on the same seeded inputs.
Indexing and tile selection are compared bit-exactly; bf16 outputs to max relative error 1e-2."""
import numpy as np
import pytest
import torch

import mortar_amd
from mortar_amd import ops, synth
from oracle import mortar_oracle as O
from util import assert_close_bf16, oracle_spmm, to_dev, to_np

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------------------------------------- committed fixtures

def test_golden_fixtures(dev):
    """The HIP path against the committed vectors (tests/golden): config 0 whole and an MLP slice with gating."""
    import golden_util as G
    z = G.load("c0_spmm.npz")
    m = G.matrix(z)
    W = synth.to_pack(m, dev)
    x = torch.from_numpy(z["x_bits"].view(np.int16)).view(torch.bfloat16).to(dev)
    ref = O.bf16_from_bits(z["y_bits"])
    assert_close_bf16(to_np(ops.spmm(x, W)), ref, "c0 spmm (64 rows)")
    assert_close_bf16(to_np(ops.spmm(x[:3], W)), ref[:3], "c0 spmm (3 rows, decode tile)")
    z = G.load("mlp_slice.npz")
    Wgu, Wdn = synth.to_pack(G.matrix(z, "gate_up_"), dev), synth.to_pack(G.matrix(z, "down_"), dev)
    x = torch.from_numpy(z["x_bits"].view(np.int16)).view(torch.bfloat16).to(dev)
    logits = torch.from_numpy(z["logits_bits"].view(np.float32)).to(dev)
    gates, active = ops.remoe_gates(logits, 11)
    assert np.array_equal(active.cpu().numpy(), z["active"])                       # tile selection bit-exact
    np.testing.assert_allclose(gates.cpu().numpy(), z["gates_bits"].view(np.float32), rtol=2e-6, atol=0)
    h = ops.gateup_swiglu(x, Wgu)
    assert_close_bf16(to_np(h), O.bf16_from_bits(z["h_bits"]), "h", ulps=4)
    assert_close_bf16(to_np(ops.spmm(h, Wdn)), O.bf16_from_bits(z["y_bits"]), "y", ulps=8)
    route = ops.remoe_route(active, ops.route_tile(Wgu, 8))
    hr = ops.gateup_swiglu(x, Wgu, gates=gates, route=route)
    yr = ops.spmm(hr, Wdn, active=active)
    assert_close_bf16(to_np(yr), O.bf16_from_bits(z["y_routed_bits"]), "y routed", ulps=8)


# ---------------------------------------------------------------------------------------------- prefill SpMM

def test_c0_single_spmm(dev):
    """benchmark config 0: x 64x768, W 768->2048, 25 % uniform, ternary p=(.3,.4,.3), scale U(.01,.1)."""
    m = synth.synth_matrix(2048, 768, 0.25, seed=100)
    x = synth.synth_x(64, 768, seed=101)
    W = synth.to_pack(m, dev)
    for fn in (ops.spmm, ops.gemv):
        y = to_np(fn(to_dev(x, dev), W))
        assert_close_bf16(y, oracle_spmm(x, m), fn.__name__)


@pytest.mark.parametrize("M", [1, 15, 16, 17, 100, 128, 129, 300])
def test_spmm_ragged_m(dev, M):
    m = synth.synth_matrix(16 * 10, 16 * 20, 0.3, seed=M)
    x = synth.synth_x(M, 320, seed=M + 1)
    y = to_np(ops.spmm(to_dev(x, dev), synth.to_pack(m, dev)))
    assert_close_bf16(y, oracle_spmm(x, m), f"M={M}")


@pytest.mark.parametrize("shape,density,zipf", [((16, 16), 1.0, None), ((16 * 3, 16 * 29), 0.1, None),
                                                 ((16 * 37, 16 * 15), 1.0, None), ((16 * 40, 16 * 60), 0.25, 1.2),
                                                 ((16 * 5, 16 * 352), 0.25, 1.2)])
def test_spmm_shapes(dev, shape, density, zipf):
    m = synth.synth_matrix(shape[0], shape[1], density, seed=7, zipf_s=zipf)
    x = synth.synth_x(200, shape[1], seed=8)
    y = to_np(ops.spmm(to_dev(x, dev), synth.to_pack(m, dev)))
    assert_close_bf16(y, oracle_spmm(x, m), str(shape))


def test_spmm_exact_cases(dev):
    # identity blocks, power-of-two scales: the result is an exact scaled block permutation of x
    perm = np.array([2, 0, 3, 1], np.int16)
    m = dict(codes=np.tile(np.eye(16, dtype=np.int8), (4, 1, 1)), scales=np.array([0.5, 0.25, 2.0, 1.0], np.float32),
             col_idx=perm, row_idx=np.arange(4, dtype=np.int16), offsets=np.arange(5, dtype=np.int32), shape=(64, 64))
    x = synth.synth_x(40, 64, 3)
    y = to_np(ops.spmm(to_dev(x, dev), synth.to_pack(m, dev)))
    for r in range(4):
        assert np.array_equal(y[:, 16 * r:16 * r + 16], m["scales"][r] * x[:, 16 * perm[r]:16 * perm[r] + 16])
    # negative identity and every single (n, c) position of a block: catches any unpack bit-position slip
    for n, c, sgn in [(n, c, s) for n in (0, 5, 15) for c in range(16) for s in (1, -1)]:
        codes = np.zeros((1, 16, 16), np.int8); codes[0, n, c] = sgn
        m1 = dict(codes=codes, scales=np.array([1.0], np.float32), col_idx=np.zeros(1, np.int16),
                  row_idx=np.zeros(1, np.int16), offsets=np.array([0, 1], np.int32), shape=(16, 16))
        xx = synth.synth_x(16, 16, 5)
        yy = to_np(ops.spmm(to_dev(xx, dev), synth.to_pack(m1, dev)))
        want = np.zeros((16, 16), np.float32); want[:, n] = sgn * xx[:, c]
        assert np.array_equal(yy, want), (n, c, sgn)


def test_spmm_noncontiguous_input_and_errors(dev):
    m = synth.synth_matrix(64, 128, 0.5, 1)
    W = synth.to_pack(m, dev)
    x = synth.synth_x(50, 256, 2)
    xt = to_dev(x, dev)[:, ::2]                                   # strided view -> made contiguous by the wrapper
    assert_close_bf16(to_np(ops.spmm(xt, W)), oracle_spmm(np.ascontiguousarray(x[:, ::2]), m))
    with pytest.raises(ValueError):
        ops.spmm(to_dev(x, dev), W)                               # wrong feature count
    with pytest.raises(TypeError):
        ops.spmm(to_dev(x[:, :128], dev).float(), W)


def test_stk_dds_operator_signature(dev):
    m = synth.synth_matrix(128, 96, 0.5, 11)
    data = torch.from_numpy(O.effective_blocks(m["codes"], m["scales"])).to(torch.bfloat16).to(dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    z16, z32 = torch.zeros(1, dtype=torch.int16, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)
    x = synth.synth_x(70, 96, 12)
    y = mortar_amd.stk_dds(to_dev(x, dev), data, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32,
                           96, 128, True)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (70, 128)
    assert_close_bf16(to_np(y), oracle_spmm(x, m))
    with pytest.raises(ValueError, match="int16"):
        mortar_amd.stk_dds(to_dev(x, dev), data, t(m["offsets"]), t(m["row_idx"]).int(), t(m["col_idx"]), z32, z16, z32, 96, 128, True)
    # any block values, as the reference's operator: random bf16 data against the dense float64 product
    rnd = torch.randn_like(data)
    yr = mortar_amd.stk_dds(to_dev(x, dev), rnd, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, 96, 128, True)
    dense = O.to_dense(rnd.float().cpu().numpy(), m["row_idx"], m["col_idx"], (128, 96)).astype(np.float64)
    assert_close_bf16(to_np(yr), (O.bf16_round(x).astype(np.float64) @ dense.T).astype(np.float32), "stk_dds, arbitrary values")
    from mortar_amd.stk import stk_dds_ternary
    yt = stk_dds_ternary(to_dev(x, dev), data, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, 96, 128, True)
    assert_close_bf16(to_np(yt), oracle_spmm(x, m), "stk_dds_ternary")
    with pytest.raises(ValueError, match="ternary"):
        stk_dds_ternary(to_dev(x, dev), rnd, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, 96, 128, True)


@pytest.mark.parametrize("out_f,in_f,M,density,zipf", [(16 * 8, 16 * 6, 70, 0.5, None), (2048, 768, 64, 0.25, None),
                                                       (16 * 40, 2048, 333, 0.25, 1.2), (16 * 12, 16 * 352, 200, 0.25, 1.2),
                                                       (16 * 70, 16 * 400, 37, 0.1, None), (16 * 3, 16 * 3, 1, 1.0, None)])
def test_dds_values_any_block_values(dev, out_f, in_f, M, density, zipf):
    """The product over stored bf16 block values (what stk_dds calls) against the dense float64 product of the scattered
    matrix: one K segment and several (in_features > 2480), ragged rows, odd block counts, M below and above one token
    tile, both orientations; 1e-2 / bf16 rounding bar as for the ternary kernels."""
    m = synth.synth_matrix(out_f, in_f, density, seed=out_f + in_f, zipf_s=zipf)
    nnz = m["col_idx"].size
    rng = np.random.default_rng(nnz)
    vals = O.bf16_round((rng.standard_normal((nnz, 16, 16)) * rng.uniform(0.01, 2.0, (nnz, 1, 1))).astype(np.float32))
    dense = O.to_dense(vals, m["row_idx"], m["col_idx"], (out_f, in_f)).astype(np.float64)
    from mortar_amd.pack import BcsrTopology
    T = BcsrTopology(m["offsets"], m["col_idx"], out_f, in_f, dev)
    assert (T.nseg > 1) == (in_f // 16 > 155)
    data = torch.from_numpy(vals).to(torch.bfloat16).to(dev)
    x = synth.synth_x(M, in_f, seed=5)
    y = ops.dds_values(to_dev(x, dev), data, T)
    assert_close_bf16(to_np(y), (x.astype(np.float64) @ dense.T).astype(np.float32), "values product", ulps=4)
    Tt, src = T.transposed()
    dy = synth.synth_x(M, out_f, seed=6)
    dx = ops.dds_values(to_dev(dy, dev), data[src].transpose(1, 2).contiguous(), Tt)
    assert_close_bf16(to_np(dx), (dy.astype(np.float64) @ dense).astype(np.float32), "values product, W^T", ulps=4)
    z16, z32 = torch.zeros(1, dtype=torch.int16, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    y2 = mortar_amd.stk_dds(to_dev(x, dev), data, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, in_f, out_f, True)
    assert torch.equal(y2, y)
    dx2 = mortar_amd.stk_dds(to_dev(dy, dev), data, t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, out_f, in_f, False)
    assert torch.equal(dx2, dx)
    with pytest.raises(TypeError):
        ops.dds_values(to_dev(x, dev), data.float(), T)


# ---------------------------------------------------------------------------------------------- SwiGLU MLP

@pytest.mark.parametrize("M", [64, 200])
def test_mlp_base_config_slice(dev, M):
    """benchmark config 1 shapes (d_model 768, d_ff 2048) on a token slice the oracle finishes quickly."""
    spec = synth.synth_mlp(768, 2048, 0.25, seed=20)
    x = synth.synth_x(M, 768, 21)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    h = ops.gateup_swiglu(to_dev(x, dev), Wgu)
    assert_close_bf16(to_np(h), ref["h"], "h", ulps=4)
    y = ops.spmm(h, Wdn)
    assert_close_bf16(to_np(y), ref["y"], "y", ulps=8)
    mlp = synth.mlp_module(spec, dev)
    y2 = mlp(to_dev(x, dev).reshape(2, M // 2, 768))
    assert tuple(y2.shape) == (2, M // 2, 768) and y2.dtype == torch.bfloat16
    assert torch.equal(y2.reshape(M, 768), y) or M <= 64          # same kernels for M > 64
    assert_close_bf16(to_np(y2).reshape(M, 768), ref["y"], "module", ulps=8)


@pytest.mark.parametrize("d_model,d_ff,M,zipf", [(2048, 5632, 4096, None), (2048, 5632, 1000, 1.2), (768, 2048, 1200, None),
                                                 (256, 16 * 40, 600, 1.2), (2048, 5632, 513, None), (2048, 5632, 300, None),
                                                 (16 * 30, 16 * 352, 530, None)])
def test_mlp_one_call_equals_the_two_calls(dev, d_model, d_ff, M, zipf):
    """mortar_mlp_bf16 (hidden activations in the library's own layout: tile order from 513 rows, with the asynchronous
    stage-in of `down`) gives the same bits as gate_up + SwiGLU followed by the plain product: plain, with cluster gates,
    with the RMSNorm folded in, in two phases, with a reused workspace; and meets the oracle on sampled rows."""
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=40, zipf_s=zipf)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    x = synth.synth_x(M, d_model, 41)
    xd = to_dev(x, dev)
    ncl = d_ff // 16
    gates, _ = ops.remoe_gates(torch.from_numpy(synth.synth_logits(M, ncl, 42)).to(dev), ncl // 4)
    nw = torch.from_numpy(O.bf16_round(1 + 0.1 * np.random.default_rng(43).standard_normal(d_model).astype(np.float32))).to(torch.bfloat16).to(dev)
    ws = torch.full((ops.mlp_hidden_bytes(M, d_ff),), 0xFF, dtype=torch.uint8, device=dev)      # NaN patterns: rows past M stay so
    for g, nm in ((None, None), (gates, None), (None, (nw, 1e-6)), (gates, (None, 1e-6))):
        if nm is not None and not ops.norm_fusable(Wgu):
            continue
        want = ops.spmm(ops.gateup_swiglu(xd, Wgu, gates=g, norm=nm), Wdn)
        assert torch.equal(ops.mlp(xd, Wgu, Wdn, gates=g, norm=nm), want)
        assert torch.equal(ops.mlp(xd, Wgu, Wdn, gates=g, norm=nm, hidden=ws), want)
        y = torch.full_like(want, float("nan"))
        ops.mlp(xd, Wgu, Wdn, gates=g, norm=nm, hidden=ws, out=y, phase=1)
        assert bool(torch.isnan(y).all())                                   # phase 1 writes the workspace only
        ops.mlp(xd, Wgu, Wdn, gates=g, norm=nm, hidden=ws, out=y, phase=2)
        assert torch.equal(y, want)
    rows = np.random.default_rng(44).choice(M, 24, replace=False)
    ref = O.swiglu_mlp(x[rows], spec["gate_up"], spec["down"])
    assert_close_bf16(to_np(ops.mlp(xd, Wgu, Wdn))[rows], ref["y"], "one-call MLP vs oracle", ulps=8)
    with pytest.raises(ValueError):
        ops.mlp(xd, Wgu, Wdn, hidden=ws[:16])
    with pytest.raises(ValueError):
        ops.mlp(xd, Wdn, Wgu)


def test_mlp_with_gates_and_skip(dev):
    """ReMoE-routed MLP: cluster size 16 (one block-row per cluster), k-th threshold gating, tile skipping."""
    d_model, d_ff, M, ncl, k = 256, 16 * 40, 300, 40, 10
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=30)
    x = synth.synth_x(M, d_model, 31)
    logits = synth.synth_logits(M, ncl, 32)
    g_ref, act_ref = O.remoe_gates(logits, k)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
    gates, active = ops.remoe_gates(torch.from_numpy(logits).to(dev), k)
    assert np.array_equal(active.cpu().numpy().astype(bool), act_ref)           # tile selection bit-exact
    np.testing.assert_allclose(gates.cpu().numpy(), g_ref, rtol=2e-6, atol=0)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    xd = to_dev(x, dev)
    h_dense = ops.gateup_swiglu(xd, Wgu, gates=gates)
    assert_close_bf16(to_np(h_dense), ref["h"], "h gated", ulps=4)
    cnt, lst = ops.remoe_route(active, ops.route_tile(Wgu, M))
    h_skip = torch.full_like(h_dense, float("nan"))                             # untouched entries stay NaN
    ops.gateup_swiglu(xd, Wgu, gates=gates, route=(cnt, lst), out=h_skip)
    hs, hd = to_np(h_skip), to_np(h_dense)
    on = np.repeat(act_ref, 16, axis=1)
    assert np.array_equal(hs[on], hd[on]) and np.isnan(hs[~on]).all()           # exactly the active tiles written
    y = ops.spmm(h_skip, Wdn, active=active)
    assert_close_bf16(to_np(y), ref["y"], "y routed", ulps=8)
    mlp = synth.mlp_module(spec, dev)
    y2 = mlp(xd, gates=gates)
    assert torch.equal(y2, y)


@pytest.mark.parametrize("route_skip", [False, True])
def test_routed_module_mask_follows_the_call(dev, route_skip):
    """The carved routed forward takes its tile mask from the gates of the current call: a no-grad call with 128 rows
    followed by a grad-enabled call with 32 other rows (router parameters trainable, weights packed) must route the
    second call by its own gates, not by what the first call left in the router.  Both prefill forms: gates in the
    gate_up epilogue (the default) and token lists + routed gate_up + masked down (route_skip)."""
    d_model, d_ff, ncl = 256, 16 * 40, 40
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=33)
    mlp = synth.mlp_module(spec, dev)
    assert mlp.route_skip is False
    mlp.route_skip = route_skip
    mlp.enable_routing(n_clusters=ncl, activation_ratio=0.25, n_iters=1)
    torch.manual_seed(5)
    with torch.no_grad():
        mlp.router.group_bias.copy_(torch.randn(ncl, device=dev))
    def oracle_for(x):
        with torch.no_grad():
            lg = mlp.router.group_logits(to_dev(x, dev), 0).float().cpu().numpy()
        g_ref, a_ref = O.remoe_gates(lg, mlp.router.activation_k)
        return O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)["y"], a_ref
    xa, xb = synth.synth_x(128, d_model, 34), synth.synth_x(32, d_model, 35)
    with torch.no_grad():
        ya = mlp(to_dev(xa, dev))
    ref_a, act_a = oracle_for(xa)
    assert_close_bf16(to_np(ya), ref_a, "no-grad call", ulps=8)
    assert mlp.router.last_active.shape == (128, ncl)
    assert any(p.requires_grad for p in mlp.router.parameters()) and torch.is_grad_enabled()
    yb = mlp(to_dev(xb, dev))                                  # grad mode on, x and the packed weights need none
    ref_b, act_b = oracle_for(xb)
    assert not np.array_equal(act_a[:32], act_b)
    assert_close_bf16(to_np(yb), ref_b, "grad-enabled call after a larger no-grad call", ulps=8)
    assert mlp.router.last_active.shape == (32, ncl)
    assert np.array_equal(mlp.router.last_active.cpu().numpy().astype(bool), act_b)


@pytest.mark.parametrize("d_model,d_ff", [(256, 16 * 40), (2048, 16 * 24), (16 * 30, 16 * 352)])
def test_prefill_code_streams_agree(dev, d_model, d_ff):
    """Prefill kernels over the 4-bit code stream and over the 2-bit one do the same arithmetic: identical bits
    (64- and 32-token resident tiles, K-segmented `down`; plain, gated + routed, masked)."""
    M, ncl = 200, d_ff // 16
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=33, zipf_s=1.2)
    xd = to_dev(synth.synth_x(M, d_model, 34), dev)
    gates, active = ops.remoe_gates(torch.from_numpy(synth.synth_logits(M, ncl, 35)).to(dev), ncl // 4)
    outs = []
    for stream in (True, False):
        Wgu, Wdn = (synth.to_pack(spec[k], dev, prefill_stream=stream) for k in ("gate_up", "down"))
        assert (Wgu.codes4_o is not None) == stream
        h = ops.gateup_swiglu(xd, Wgu)
        res = [h, ops.spmm(h, Wdn)]
        tile = ops.route_tile(Wgu, M)
        if tile:
            hr = torch.zeros_like(h)
            ops.gateup_swiglu(xd, Wgu, gates=gates, route=ops.remoe_route(active, tile), out=hr)
            res += [hr, ops.spmm(hr, Wdn, active=active)]
        outs.append(res)
    assert_close_bf16(to_np(outs[0][1]), O.swiglu_mlp(synth.synth_x(M, d_model, 34), spec["gate_up"], spec["down"])["y"], "y", ulps=8)
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("seg_cb", [7, 32, 64])
@pytest.mark.parametrize("M", [5, 16, 100, 300])
def test_narrow_k_segments(dev, seg_cb, M):
    """A pack built with narrow K segments (MortarPack(seg_cb=...)) walks several segments per row in every kernel
    family (prefill tiles run the K-segmented kernel also for gate_up, decode tiles walk the segments back to back):
    same products as the oracle, and the padding blocks between a row's segments contribute nothing."""
    from mortar_amd.pack import MortarPack
    d_model, d_ff = 16 * 72, 16 * 40
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=71, zipf_s=1.2)
    x = synth.synth_x(M, d_model, 72)
    xd = to_dev(x, dev)
    def pk(m):
        return MortarPack(synth.flat_pack(m["codes"]), m["scales"], m["col_idx"], m["offsets"], m["shape"][0], m["shape"][1],
                          dev, seg_cb=seg_cb)
    Wgu, Wdn = pk(spec["gate_up"]), pk(spec["down"])
    assert Wgu.nseg == -(-(d_model // 16) // seg_cb) and Wdn.nseg == -(-(d_ff // 16) // seg_cb)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    h = ops.gateup_swiglu(xd, Wgu)
    assert_close_bf16(to_np(h), ref["h"], "h", ulps=8)
    assert_close_bf16(to_np(ops.spmm(h, Wdn)), oracle_spmm(to_np(h), spec["down"]), "y", ulps=8)
    assert_close_bf16(to_np(ops.spmm(xd, Wgu)), oracle_spmm(x, spec["gate_up"]), "gu", ulps=8)


@pytest.mark.parametrize("d_model,seg_cb,M", [(16 * 30, 20, 257), (16 * 200, None, 4), (2048, 32, 17), (16 * 78, 65, 63)])
def test_routed_gate_up_over_several_k_segments(dev, d_model, seg_cb, M):
    """Routed skipping whenever mortar_route_tile() names a tile, also for a matrix whose stream has several K segments
    (a narrow seg_cb, or in_features wider than one prefill segment at a decode-sized M): exactly the active tiles are
    written and they equal the dense gated call."""
    from mortar_amd.pack import MortarPack
    d_ff, ncl = 16 * 22, 22
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=91)
    m = spec["gate_up"]
    Wgu = MortarPack(synth.flat_pack(m["codes"]), m["scales"], m["col_idx"], m["offsets"], m["shape"][0], m["shape"][1], dev,
                     seg_cb=seg_cb)
    assert Wgu.nseg > 1
    x = synth.synth_x(M, d_model, 92)
    logits = synth.synth_logits(M, ncl, 93)
    g_ref, act_ref = O.remoe_gates(logits, 7)
    gates, active = ops.remoe_gates(torch.from_numpy(logits).to(dev), 7)
    xd = to_dev(x, dev)
    h_dense = ops.gateup_swiglu(xd, Wgu, gates=gates)
    assert_close_bf16(to_np(h_dense), O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)["h"], "h gated", ulps=8)
    tile = ops.route_tile(Wgu, M)
    assert tile > 0
    h_skip = torch.full_like(h_dense, float("nan"))
    ops.gateup_swiglu(xd, Wgu, gates=gates, route=ops.remoe_route(active, tile), out=h_skip)
    hs, hd, on = to_np(h_skip), to_np(h_dense), np.repeat(act_ref, 16, axis=1)
    assert np.array_equal(hs[on], hd[on]) and np.isnan(hs[~on]).all()


@pytest.mark.parametrize("d_model,d_ff,M", [(256, 16 * 40, 200), (2048, 16 * 24, 130), (16 * 30, 16 * 352, 100),
                                            (256, 16 * 40, 1), (2048, 16 * 24, 5), (16 * 30, 16 * 352, 16), (768, 2048, 40)])
def test_one_scale_per_matrix(dev, d_model, d_ff, M):
    """Matrices with one scale (the reference's per-tensor mortar_scale): the kernels that scale the fp32 sums once
    against the oracle and against the per-block kernels on the same data (plain, gated, routed, masked), for the
    prefill tiles, the K-segmented `down`, the decode tiles and a layer-batched launch."""
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=77, zipf_s=1.2)
    spec["gate_up"]["scales"] = np.float32(0.0437)
    spec["down"]["scales"] = np.float32(0.0291)
    x = synth.synth_x(M, d_model, 78)
    xd = to_dev(x, dev)
    ncl = d_ff // 16
    gates, active = ops.remoe_gates(torch.from_numpy(synth.synth_logits(M, ncl, 79)).to(dev), ncl // 4)
    outs = []
    for after in (True, False):
        Wgu, Wdn = (synth.to_pack(spec[k], dev, scale_after_sum=after) for k in ("gate_up", "down"))
        assert (Wgu.uniform_scale != 0) == after and (Wdn.uniform_scale != 0) == after
        h = ops.gateup_swiglu(xd, Wgu)
        res = [h, ops.spmm(h, Wdn), ops.gateup_swiglu(xd, Wgu, gates=gates)]
        tile = ops.route_tile(Wgu, M)
        if tile:
            hr = torch.zeros_like(h)
            ops.gateup_swiglu(xd, Wgu, gates=gates, route=ops.remoe_route(active, tile), out=hr)
            res += [hr, ops.spmm(hr, Wdn, active=active)]
        if M <= 16:
            hs = [torch.empty_like(h) for _ in range(3)]
            ops.LayerStack([Wgu] * 3, [xd] * 3, hs, swiglu=True).run()
            res += hs[1:2]
        outs.append(res)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    assert_close_bf16(to_np(outs[0][0]), ref["h"], "h", ulps=4)
    assert_close_bf16(to_np(outs[0][1]), ref["y"], "y", ulps=8)
    for a, b in zip(*outs):
        assert_close_bf16(to_np(a), to_np(b).astype(np.float32), "scale after sum vs per block", ulps=8)


def test_remoe_route_lists_exact(dev):
    rng = np.random.default_rng(40)
    act = (rng.random((333, 70)) < 0.25).astype(np.uint8)
    act[:128, 3] = 0; act[128:256, 5] = 1
    cnt, lst = ops.remoe_route(torch.from_numpy(act).to(dev), 128)
    cnt, lst = cnt.cpu().numpy(), lst.cpu().numpy()
    for t in range(3):
        for c in range(70):
            want = np.nonzero(act[t * 128:(t + 1) * 128, c])[0]
            assert cnt[t, c] == len(want) and np.array_equal(lst[t, c, :len(want)], want)


def test_remoe_gates_ties_and_edges(dev):
    rng = np.random.default_rng(41)
    for n, k in ((8, 3), (16, 8), (352, 88), (100, 100), (65, 1), (1024, 256)):
        lg = rng.integers(-3, 4, size=(257, n)).astype(np.float32)
        lg[0] = 1.0; lg[1, 0] = -0.0; lg[1, 1] = 0.0
        g_ref, a_ref = O.remoe_gates(lg, k)
        g, a = ops.remoe_gates(torch.from_numpy(lg).to(dev), k)
        assert np.array_equal(a.cpu().numpy().astype(bool), a_ref), (n, k)
        np.testing.assert_allclose(g.cpu().numpy(), g_ref, rtol=3e-6, atol=0)
    # the clamp of the gate sum at 1e-6 (routing.py:253): one entry one fp32 ulp above the k-th -> 2^-23 * 2e6
    lg = np.array([[1.0 + 2.0 ** -23, 1.0, 0.0, -1.0], [1.0 + 2.0 ** -19, 1.0, 0.0, -1.0]], np.float32)
    g, a = ops.remoe_gates(torch.from_numpy(lg).to(dev), 2)
    np.testing.assert_allclose(g.cpu().numpy(), [[0.23841858, 0, 0, 0], [2.0, 0, 0, 0]], rtol=1e-6, atol=0)
    assert a.cpu().numpy().astype(bool).tolist() == [[True, False, False, False]] * 2
    lg = synth.synth_logits(4096, 352, 42)                                      # benchmark config 3 router
    g_ref, a_ref = O.remoe_gates(lg, 88)
    g, a = ops.remoe_gates(torch.from_numpy(lg).to(dev), 88)
    assert np.array_equal(a.cpu().numpy().astype(bool), a_ref) and (a_ref.sum(1) == 87).all()
    with pytest.raises(ValueError):
        ops.remoe_gates(torch.zeros(2, 2000, device=dev), 5)


@pytest.mark.parametrize("B,d,nsk,n,xdt", [(1, 256, 4, 16, "bf16"), (5, 768, 4, 16, "bf16"), (16, 2048, 8, 64, "bf16"),
                                          (3, 2048, 18, 352, "f32"), (64, 512, 4, 16, "f32"), (2, 264, 3, 9, "bf16"),
                                          (2, 2048, 19, 352, "bf16"), (5, 256, 5, 20, "f32"), (1, 512, 33, 1024, "f32")])
def test_fused_router_front_end(dev, B, d, nsk, n, xdt):
    """Two-launch decode router (projection; LayerNorm + product keys + gating tail) against the float64 oracle:
    logits to fp32 rounding, the active set exactly except where a logit sits within rounding of the threshold,
    gates to 1e-4; and against the torch ops of TileRouter.group_logits + the stand-alone gates kernel."""
    rng = np.random.default_rng(70 + B)
    k = max(1, n // 4)
    x = O.bf16_round(rng.standard_normal((B, d)).astype(np.float32)) if xdt == "bf16" else rng.standard_normal((B, d)).astype(np.float32)
    wq = (rng.standard_normal((d, d)) / np.sqrt(d)).astype(np.float32); it = (0.1 * rng.standard_normal(d)).astype(np.float32)
    lw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32); lb = (0.1 * rng.standard_normal(d)).astype(np.float32)
    ka = (rng.standard_normal((nsk, d // 2)) / np.sqrt(d // 2)).astype(np.float32)
    kb = (rng.standard_normal((nsk, d // 2)) / np.sqrt(d // 2)).astype(np.float32)
    bias = (0.1 * rng.standard_normal(n)).astype(np.float32)
    T = lambda a: torch.from_numpy(a).to(dev)
    xd = to_dev(x, dev) if xdt == "bf16" else T(x)
    gates, active, logits = ops.router_fused(xd, T(wq), T(it), T(lw), T(lb), 1e-5, T(ka), T(kb), T(bias), k, want_logits=True)
    ref = O.router_logits(x, wq, it, lw, lb, 1e-5, ka, kb, bias)
    np.testing.assert_allclose(logits.cpu().numpy(), ref, rtol=0, atol=2e-5 * max(1.0, np.abs(ref).max()))
    g_ref, a_ref = O.remoe_gates(ref.astype(np.float32), k)
    kth = O.kth_largest(ref.astype(np.float32), k)[:, None] if k < n else np.full((B, 1), -np.inf)
    clear = np.abs(ref - kth) > 1e-4                       # logits not within rounding of the threshold
    assert np.array_equal(active.cpu().numpy().astype(bool)[clear], a_ref[clear])
    np.testing.assert_allclose(gates.cpu().numpy(), g_ref, rtol=0, atol=2e-4)
    # the fused tail equals the stand-alone gates kernel on the fused logits, bit for bit
    g2, a2 = ops.remoe_gates(logits, k)
    assert torch.equal(g2, gates) and torch.equal(a2, active)
    # module path: TileRouter picks the fused router for decode-sized inference calls
    from mortar_amd.routing import TileRouter
    rt = TileRouter(n, d, activation_ratio=k / n, n_sub_keys=nsk, n_iters=2).to(dev)
    with torch.no_grad():
        rt.query_proj.weight.copy_(T(wq)); rt.iter_embed[1].copy_(T(it)); rt.query_norm.weight.copy_(T(lw))
        rt.query_norm.bias.copy_(T(lb)); rt.sub_keys_a.copy_(T(ka)); rt.sub_keys_b.copy_(T(kb)); rt.group_bias.copy_(T(bias))
        assert rt.activation_k == k and rt._fused_ok(xd)
        gm, _ = rt(xd, iter_idx=1)
        assert torch.equal(gm, gates)
        lt = rt.group_logits(xd, 1)                       # eager torch ops (library GEMMs)
    np.testing.assert_allclose(lt.cpu().numpy(), ref, rtol=0, atol=2e-5 * max(1.0, np.abs(ref).max()))


@pytest.mark.parametrize("N,d,nsk,n", [(65, 256, 4, 16), (200, 768, 4, 16), (513, 2048, 19, 352), (300, 2048, 8, 64),
                                       (130, 264, 3, 20), (70, 512, 32, 1000), (100, 4096, 4, 16), (33, 8192, 5, 25), (3, 512, 4, 16),
                                       (66, 256, 23, 500)])
def test_router_tail_behind_a_library_projection(dev, N, d, nsk, n):
    """Prefill-sized router: the dense query projection through the library, then ONE launch for LayerNorm, sub-key
    scores, product-key logits (direct, wrapped and ranked branches) and the gating tail, against the float64 oracle (same
    bars as the two-launch decode router) and against the module's eager torch ops."""
    rng = np.random.default_rng(170 + N)
    k = max(1, n // 4)
    x = O.bf16_round(rng.standard_normal((N, d)).astype(np.float32))
    wq = (rng.standard_normal((d, d)) / np.sqrt(d)).astype(np.float32); it = (0.1 * rng.standard_normal(d)).astype(np.float32)
    lw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32); lb = (0.1 * rng.standard_normal(d)).astype(np.float32)
    ka = (rng.standard_normal((nsk, d // 2)) / np.sqrt(d // 2)).astype(np.float32)
    kb = (rng.standard_normal((nsk, d // 2)) / np.sqrt(d // 2)).astype(np.float32)
    bias = (0.1 * rng.standard_normal(n)).astype(np.float32)
    T = lambda a: torch.from_numpy(a).to(dev)
    xd = to_dev(x, dev)
    qv = torch.nn.functional.linear(xd.float(), T(wq))
    gates, active, logits = ops.router_tail(qv, T(it), T(lw), T(lb), 1e-5, T(ka), T(kb), T(bias), k, want_logits=True)
    ref = O.router_logits(x, wq, it, lw, lb, 1e-5, ka, kb, bias)
    np.testing.assert_allclose(logits.cpu().numpy(), ref, rtol=0, atol=2e-5 * max(1.0, np.abs(ref).max()))
    g_ref, a_ref = O.remoe_gates(ref.astype(np.float32), k)
    kth = O.kth_largest(ref.astype(np.float32), k)[:, None] if k < n else np.full((N, 1), -np.inf)
    clear = np.abs(ref - kth) > 1e-4                       # logits not within rounding of the threshold
    assert np.array_equal(active.cpu().numpy().astype(bool)[clear], a_ref[clear])
    rows = clear.all(axis=1)                                # a token with a logit at the threshold may normalise differently
    np.testing.assert_allclose(gates.cpu().numpy()[rows], g_ref[rows], rtol=0, atol=2e-4)
    g2, a2 = ops.remoe_gates(logits, k)                     # the fused tail is the stand-alone gates kernel on its own logits
    assert torch.equal(g2, gates) and torch.equal(a2, active)
    # a strided qv (rows of a wider buffer) and no iteration vector
    wide = torch.zeros((N, d + 8), dtype=torch.float32, device=dev)
    wide[:, :d] = qv + T(it)
    g3, a3 = ops.router_tail(wide[:, :d], None, T(lw), T(lb), 1e-5, T(ka), T(kb), T(bias), k)
    assert torch.equal(g3, gates) and torch.equal(a3, active)
    from mortar_amd.routing import TileRouter
    rt = TileRouter(n, d, activation_ratio=k / n, n_sub_keys=nsk, n_iters=2).to(dev)
    with torch.no_grad():
        rt.query_proj.weight.copy_(T(wq)); rt.iter_embed[1].copy_(T(it)); rt.query_norm.weight.copy_(T(lw))
        rt.query_norm.bias.copy_(T(lb)); rt.sub_keys_a.copy_(T(ka)); rt.sub_keys_b.copy_(T(kb)); rt.group_bias.copy_(T(bias))
        assert rt.activation_k == k and rt._tail_ok(xd)
        if N > ops.ROUTER_MAX_TOKENS:
            gm, am = rt.route(xd, iter_idx=1)
            assert torch.equal(gm, gates) and torch.equal(am, active)
            gf, _ = rt(xd, iter_idx=1)
            assert torch.equal(gf, gates) and torch.equal(rt.last_active, active)
        lt = rt.group_logits(xd, 1)                       # eager torch ops
    np.testing.assert_allclose(lt.cpu().numpy(), ref, rtol=0, atol=2e-5 * max(1.0, np.abs(ref).max()))
    with pytest.raises(TypeError):
        ops.router_tail(qv.double(), None, T(lw), T(lb), 1e-5, T(ka), T(kb), T(bias), k)
    if N == 3:      # more than 1024 product keys to rank: refused, the module keeps its eager path for such a router
        k33 = T((rng.standard_normal((33, d // 2))).astype(np.float32))
        with pytest.raises(ValueError):
            ops.router_tail(qv, None, T(lw), T(lb), 1e-5, k33, k33, T(np.zeros(1024, dtype=np.float32)), 5)
        assert not TileRouter(1024, d, n_sub_keys=33).to(dev)._tail_ok(xd)


def test_decode_view_of_a_segmented_matrix(dev):
    """A matrix whose prefill stream has several K segments (`down`) carries a one-segment decode stream for calls of up to
    4 rows.  The layer-batched launch picks it by itself (same results to the usual bar: the pairing of blocks into MFMAs
    follows the segments); more rows on it are refused; a matrix with one segment or device-rewritten values has none."""
    spec = synth.synth_mlp(512, 16 * 352, 0.25, seed=91, zipf_s=1.2)
    m = spec["down"]
    W = synth.to_pack(m, dev)
    assert W.nseg == 3 and synth.to_pack(spec["gate_up"], dev).decode_view(1) is None and W.decode_view(5) is None
    V = W.decode_view(3)
    assert V.nseg == 1 and V.decode_rows == 4 and V is W.decode_view(1)
    assert V.codes_o.numel() <= W.codes_o.numel()                      # one part per row: padded to octets once
    for B in (1, 3, 4, 5):
        x = synth.synth_x(B, 16 * 352, 92 + B)
        xd = to_dev(x, dev)
        ref = oracle_spmm(x, m)
        ys = [torch.empty((B, 512), dtype=torch.bfloat16, device=dev) for _ in range(3)]
        st = ops.LayerStack([W, W.clone_weights(), W], [xd] * 3, ys, swiglu=False)
        assert all(p.decode_rows == (4 if B <= 4 else 0) for p in st.packs)
        st.run()
        for y in ys:
            assert_close_bf16(to_np(y), ref, f"decode view B={B}", ulps=8)
        if B <= 4:
            assert_close_bf16(to_np(ops.spmm(xd, V)), ref, f"single launch on the decode view B={B}", ulps=8)
    with pytest.raises(ValueError):
        ops.spmm(to_dev(synth.synth_x(5, 16 * 352, 99), dev), V)            # more than 4 rows: not on this stream
    W.requantize(torch.from_numpy(O.effective_blocks(m["codes"], m["scales"])).to(dev), per_block=True)
    assert W.decode_view(1) is None                                          # the host copy of the codes is stale now
    ys = [torch.empty((2, 512), dtype=torch.bfloat16, device=dev)]
    st = ops.LayerStack([W], [to_dev(synth.synth_x(2, 16 * 352, 98), dev)], ys, swiglu=False)
    assert st.packs[0].decode_rows == 0


def test_empty_batches_launch_nothing(dev):
    """Zero rows through every operator and module of the path: empty results of the right shape, no launch, no error."""
    from mortar_amd.pack import BcsrTopology
    from mortar_amd.routing import TileRouter
    spec = synth.synth_mlp(256, 640, 0.25, seed=3)
    G, D = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    e = lambda *shape, dt=torch.bfloat16: torch.empty(shape, dtype=dt, device=dev)
    assert ops.mlp(e(0, 256), G, D).shape == (0, 256) and ops.mlp_hidden_bytes(0, 640) == 0
    assert ops.gateup_swiglu(e(0, 256), G).shape == (0, 640) and ops.spmm(e(0, 640), D).shape == (0, 256)
    m = spec["down"]
    T = BcsrTopology(m["offsets"], m["col_idx"], m["shape"][0], m["shape"][1], dev)
    assert ops.dds_values(e(0, 640), torch.zeros((T.nnz, 16, 16), dtype=torch.bfloat16, device=dev), T).shape == (0, 256)
    g, a = ops.remoe_gates(e(0, 40, dt=torch.float32), 3)
    assert g.shape == (0, 40) and a.shape == (0, 40)
    z = lambda *shape: torch.zeros(shape, device=dev)
    g, a = ops.router_tail(e(0, 256, dt=torch.float32), None, z(256), z(256), 1e-5, z(4, 128), z(4, 128), z(16), 4)
    assert g.shape == (0, 16) and a.shape == (0, 16)
    rt = TileRouter(16, 256).to(dev).eval()
    with torch.no_grad():
        assert rt(e(0, 256))[0].shape == (0, 16) and rt(torch.randn(2, 70, 256, device=dev).to(torch.bfloat16))[0].shape == (2, 70, 16)
    mlp = synth.mlp_module(spec, dev)
    assert mlp(e(0, 256)).shape == (0, 256) and mlp(e(2, 0, 256)).shape == (2, 0, 256)


def test_decode_mlp_module_routes_with_its_own_router(dev):
    """MortarDecodeMLP with a router attached (no token lists: the gated gate_up kernel leaves out inactive units
    itself) equals the step-by-step composition rmsnorm -> route -> gated gate_up -> down, and the oracle."""
    d_model, d_ff = 512, 16 * 64
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=77)
    mlp = synth.mlp_module(spec, dev)
    torch.manual_seed(5)
    mlp.enable_routing(n_clusters=16, activation_ratio=0.5, n_sub_keys=4)
    w = to_dev(O.bf16_round(1.0 + 0.1 * synth.synth_x(1, d_model, 78)[0]), dev)
    dec = mortar_amd.MortarDecodeMLP(mlp, norm_weight=w, eps=1e-6)
    for B in (1, 3, 16, 40):
        x = to_dev(synth.synth_x(B, d_model, 79 + B) * 2.0, dev)
        y = dec(x.reshape(B, 1, d_model))
        xn = ops.rmsnorm(x, w, 1e-6)
        gates, active = mlp.router.route(xn, 0)
        assert 0 < int(active.sum()) < active.numel()
        h = ops.gateup_swiglu(xn, dec.Mgu, gates=gates)
        assert torch.equal(y.reshape(B, d_model), ops.spmm(h, dec.Mdown))
        ref = O.swiglu_mlp(to_np(xn), spec["gate_up"], spec["down"], gates=gates.cpu().numpy())
        assert_close_bf16(to_np(y).reshape(B, d_model), ref["y"], f"B={B}", ulps=8)


def test_fused_router_limits(dev):
    T = lambda *s: torch.zeros(s, dtype=torch.float32, device=dev)
    x = torch.zeros((65, 64), dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="1..64 tokens"):
        ops.router_fused(x, T(64, 64), None, T(64), T(64), 1e-5, T(4, 32), T(4, 32), T(16), 4)
    with pytest.raises(ValueError, match="product keys exceed"):
        ops.router_fused(x[:2], T(64, 64), None, T(64), T(64), 1e-5, T(46, 32), T(46, 32), T(16), 4)


def test_route_flags_exact(dev):
    for ncl, d_ff in ((352, 5632), (16, 2048), (256, 2048), (44, 5632)):
        lg = synth.synth_logits(5, ncl, ncl)
        gates, _ = O.remoe_gates(lg, max(1, ncl // 4))
        r_ref, c_ref = O.route_flags(gates, d_ff)
        scratch = torch.zeros(5, 1024, dtype=torch.int32, device=dev)           # sliced scratch, as the engine does
        r, c = ops.route_flags(torch.from_numpy(gates).to(dev), d_ff, row_act=scratch[:, :2 * d_ff // 16])
        assert np.array_equal(r.cpu().numpy(), r_ref) and np.array_equal(c.cpu().numpy(), c_ref)


# ---------------------------------------------------------------------------------------------- decode

@pytest.mark.parametrize("B", [1, 4, 16, 17, 64])
def test_decode_mlp_cloud_width(dev, B):
    """benchmark config 2: d_model 2048, d_ff 5632, batch of single-token rows."""
    spec = synth.synth_mlp(2048, 5632, 0.25, seed=50)
    x = synth.synth_x(B, 2048, 51 + B)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    h = ops.gemv(to_dev(x, dev), Wgu, swiglu_out=True)
    assert_close_bf16(to_np(h), ref["h"], "h", ulps=4)
    y = ops.gemv(h, Wdn)
    assert_close_bf16(to_np(y), ref["y"], "y", ulps=8)
    gu = ops.gemv(to_dev(x, dev), Wgu)                                           # plain mode on gate_up
    assert_close_bf16(to_np(gu), ref["gu"], "gu")


@pytest.mark.parametrize("B", [1, 2, 4, 5, 16])
@pytest.mark.parametrize("dims", [(256, 16 * 44), (512, 16 * 400)])
def test_decode_small_tiles(dev, B, dims):
    """Decode batches through the SpMM entry points: 4- and 16-token tiles, K that fits LDS whole (resident)
    and K cut into segments (d_ff = 6400 > one segment), Zipf rows, per-cluster gates."""
    d_model, d_ff = dims
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=400 + B, zipf_s=1.2)
    x = synth.synth_x(B, d_model, 410 + B)
    ncl = d_ff // 16
    g_ref, _ = O.remoe_gates(synth.synth_logits(B, ncl, 420 + B), max(1, ncl // 3))
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    xd = to_dev(x, dev)
    for gates in (None, g_ref):
        ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=gates)
        gd = torch.from_numpy(gates).to(dev) if gates is not None else None
        h = ops.gateup_swiglu(xd, Wgu, gates=gd)
        assert_close_bf16(to_np(h), ref["h"], "h", ulps=4)
        y = ops.spmm(h, Wdn)
        assert_close_bf16(to_np(y), ref["y"], "y", ulps=8)
        if gates is not None:                                                        # gather-skip form
            active = (gd > 0).to(torch.uint8)
            tile = ops.route_tile(Wgu, B)
            assert tile == (4 if B <= 4 else 16)
            route = ops.remoe_route(active, tile)
            hs = torch.full_like(h, float("nan"))
            ops.gateup_swiglu(xd, Wgu, gates=gd, route=route, out=hs)
            on = np.repeat(to_np(active).astype(bool), 16, axis=1)
            assert np.array_equal(to_np(hs)[on], to_np(h)[on])
            assert np.isnan(to_np(hs)[~on]).all()
            ys = ops.spmm(hs, Wdn, active=active)
            assert_close_bf16(to_np(ys), ref["y"], "y skip", ulps=8)
    gu = ops.spmm(xd, Wgu)
    assert_close_bf16(to_np(gu), oracle_spmm(x, spec["gate_up"]), "gu")


def test_decode_gather_flags_worklist(dev):
    """The work-list GEMV with the reference's row_act / col_act gather flags (route_flags)."""
    d_model, d_ff, ncl, k, B = 512, 16 * 64, 64, 16, 3
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=70)
    x = synth.synth_x(B, d_model, 71)
    g_ref, _ = O.remoe_gates(synth.synth_logits(B, ncl, 72), k)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
    gates = torch.from_numpy(g_ref).to(dev)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    ract, cact = ops.route_flags(gates, d_ff)
    h = ops.gemv(to_dev(x, dev), Wgu, swiglu_out=True, gates=gates, row_act=ract)
    y = ops.gemv(h, Wdn, col_act=cact)
    assert_close_bf16(to_np(y), ref["y"], "flagged decode", ulps=8)


@pytest.mark.parametrize("B", [1, 5, 16, 37])
def test_decode_gather_flags_are_per_stream(dev, B):
    """Flags that do NOT follow from the gates and differ between the streams (fused_decode_step.py:1378-1393: stream b
    reads ROWACT[b, r] and COLACT[b, cb]): the bf16 work-list GEMV against the oracle with the same flags, whole rows per
    entry and split rows, with and without gates; flags_from_gates=False keeps caller flags beside gates."""
    d_model, d_ff, ncl = 512, 16 * 48, 12
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=75, zipf_s=1.2)
    gu_m, dn_m = spec["gate_up"], spec["down"]
    Wgu, Wdn = synth.to_pack(gu_m, dev), synth.to_pack(dn_m, dev)
    rng = np.random.default_rng(76 + B)
    x = synth.synth_x(B, d_model, 77)
    xd = to_dev(x, dev)
    ract_np = (rng.random((B, 2 * d_ff // 16)) < 0.6).astype(np.int32)
    ract_np[:, 2] = 0; ract_np[:, 2 + d_ff // 16] = 0                              # a unit that is off for every stream
    cact_np = (rng.random((B, d_ff // 16)) < 0.6).astype(np.int32); cact_np[:, 7] = 0
    ract, cact = torch.from_numpy(ract_np).to(dev), torch.from_numpy(cact_np).to(dev)
    sc = lambda m: O.bf16_round(m["scales"])                                       # the bf16 path multiplies bf16(scale)
    gu = O.bf16_round(O.mortar_gemv(x, gu_m["codes"], sc(gu_m), gu_m["col_idx"], gu_m["offsets"], row_act=ract_np))
    h_ref = O.swiglu(gu)
    gates_np = (rng.random((B, ncl)) * 2).astype(np.float32); gates_np[:, 1] = 0
    hg_ref = O.bf16_round(h_ref.reshape(B, ncl, -1) * O.bf16_round(gates_np)[:, :, None]).reshape(B, d_ff)
    gates = torch.from_numpy(gates_np).to(dev)
    for mb in (None, 4):
        h = ops.gemv(xd, Wgu, swiglu_out=True, row_act=ract, max_blocks=mb)
        assert_close_bf16(to_np(h), h_ref, f"row flags per stream, max_blocks={mb}", ulps=4)
        assert (to_np(h)[np.repeat((ract_np[:, :d_ff // 16] == 0) | (ract_np[:, d_ff // 16:] == 0), 16, axis=1)] == 0).all()
        hg = ops.gemv(xd, Wgu, swiglu_out=True, gates=gates, row_act=ract, max_blocks=mb, flags_from_gates=False)
        assert_close_bf16(to_np(hg), hg_ref, f"row flags beside gates, max_blocks={mb}", ulps=4)
        guo = ops.gemv(xd, Wgu, row_act=ract, max_blocks=mb)
        assert_close_bf16(to_np(guo), gu, f"plain product with row flags, max_blocks={mb}", ulps=4)
        hin = O.bf16_round(rng.standard_normal((B, d_ff)).astype(np.float32))
        y_ref = O.bf16_round(O.mortar_gemv(hin, dn_m["codes"], sc(dn_m), dn_m["col_idx"], dn_m["offsets"], col_act=cact_np))
        y = ops.gemv(to_dev(hin, dev), Wdn, col_act=cact, max_blocks=mb)
        assert_close_bf16(to_np(y), y_ref, f"column flags per stream, max_blocks={mb}", ulps=8)


@pytest.mark.parametrize("B,n_layers,d_model", [(3, 5, 256), (12, 5, 256), (2, 300, 256), (12, 300, 1024), (40, 5, 256),
                                                  (64, 40, 1024)])
def test_layer_stack_matches_single_launches(dev, B, n_layers, d_model):
    """Layer-batched launch: n layers in one launch match n separate launches (to fp32 summation order: the
    single-matrix launches split a row's K segments over several waves) and the oracle.  The last case has enough
    workgroups for the K-segmented `down` kernel to give every wave two row units."""
    d_ff = 16 * 380                                                                  # down is K-segmented
    specs = [synth.synth_mlp(d_model, d_ff, 0.25, seed=500 + i, zipf_s=1.2) for i in range(min(n_layers, 5))]
    packs = [(synth.to_pack(s["gate_up"], dev), synth.to_pack(s["down"], dev)) for s in specs]
    packs = [packs[i % len(packs)] for i in range(n_layers)]
    xs = [to_dev(synth.synth_x(B, d_model, 520 + i), dev) for i in range(n_layers)]
    hs = [torch.empty((B, d_ff), dtype=torch.bfloat16, device=dev) for _ in range(n_layers)]
    ys = [torch.empty((B, d_model), dtype=torch.bfloat16, device=dev) for _ in range(n_layers)]
    up = ops.LayerStack([p[0] for p in packs], xs, hs, swiglu=True)
    dn = ops.LayerStack([p[1] for p in packs], hs, ys, swiglu=False)
    for _ in range(2):
        up.run()
        dn.run()
    for i in range(n_layers):
        h1 = ops.gateup_swiglu(xs[i], packs[i][0])
        assert_close_bf16(to_np(hs[i]), to_np(h1), f"layer {i} h", ulps=2)
        assert_close_bf16(to_np(ys[i]), to_np(ops.spmm(hs[i], packs[i][1])), f"layer {i} y", ulps=2)
    ref = O.swiglu_mlp(to_np(xs[1]), specs[1]["gate_up"], specs[1]["down"])
    assert_close_bf16(to_np(ys[1]), ref["y"], "stack vs oracle", ulps=8)
    with pytest.raises(ValueError):
        ops.LayerStack([packs[0][0]], [to_dev(synth.synth_x(65, d_model, 1), dev)],
                       [torch.empty((65, d_ff), dtype=torch.bfloat16, device=dev)], swiglu=True)


@pytest.mark.parametrize("B", [1, 2, 3, 4, 5, 16])
def test_decode_rows_wider_than_any_resident_tile(dev, B):
    """in_features so wide (> 19904) that no 4-token tile of all K fits in LDS: up to 4 rows run 2-token tiles of all K,
    more rows the work-list kernel (K split over workgroups, partial sums combined) from gemv() and K-segmented tiles
    from the plain SpMM entry point; with an explicit split gemv() runs the work list at any batch.  Same product."""
    m = synth.synth_matrix(16 * 6, 16 * 1300, 0.1, seed=64, zipf_s=1.2)
    W = synth.to_pack(m, dev)
    assert ops.route_tile(W, 1) == 0 and W.nseg > 8
    x = synth.synth_x(B, 16 * 1300, 65)
    ref = oracle_spmm(x, m)
    assert_close_bf16(to_np(ops.gemv(to_dev(x, dev), W)), ref, "gemv", ulps=8)
    assert_close_bf16(to_np(ops.gemv(to_dev(x, dev), W, max_blocks=1 << 20)), ref, "work-list", ulps=8)
    assert_close_bf16(to_np(ops.spmm(to_dev(x, dev), W)), ref, "SpMM", ulps=8)


@pytest.mark.parametrize("B", [3, 8, 16, 40])
def test_layer_stack_gate_up_of_a_wide_model(dev, B):
    """Layer-batched gate_up + SwiGLU for d_model 5120 (no 16-token tile of all K fits): 4-token tiles up to 4 rows,
    K-segmented 16-token tiles beyond; every layer against the oracle."""
    d_model, d_ff, n = 5120, 16 * 24, 3
    specs = [synth.synth_mlp(d_model, d_ff, 0.25, seed=91 + i, zipf_s=1.2) for i in range(n)]
    packs = [synth.to_pack(sp["gate_up"], dev) for sp in specs]
    xs = [synth.synth_x(B, d_model, 95 + i) for i in range(n)]
    hs = [torch.full((B, d_ff), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(n)]
    ops.LayerStack(packs, [to_dev(x, dev) for x in xs], hs, swiglu=True).run()
    for i in range(n):
        assert_close_bf16(to_np(hs[i]), O.swiglu_mlp(xs[i], specs[i]["gate_up"], specs[i]["down"])["h"], f"layer {i} B={B}", ulps=8)


@pytest.mark.parametrize("seg_cb", [None, 8])
def test_gate_up_many_units_over_several_16_token_tiles(dev, seg_cb):
    """gate_up with 352 row units at 40 and 64 rows: three or four 16-token tiles of 88 four-unit workgroups each exceed
    one round, so 8 units of two waves share a workgroup; one K segment (two parts per unit) and two (four parts)."""
    from mortar_amd.pack import MortarPack
    d_model, d_ff, ncl = 256, 16 * 352, 352
    spec = synth.synth_mlp(d_model, d_ff, 0.5, seed=83, zipf_s=1.2)
    m = spec["gate_up"]
    Wgu = MortarPack(synth.flat_pack(m["codes"]), m["scales"], m["col_idx"], m["offsets"], m["shape"][0], m["shape"][1], dev,
                     seg_cb=seg_cb)
    assert Wgu.nseg == (1 if seg_cb is None else 2)
    for M in (40, 64):
        x = synth.synth_x(M, d_model, 84 + M)
        g_ref = O.remoe_gates(synth.synth_logits(M, ncl, 85), 88)[0]
        ref, refg = O.swiglu_mlp(x, spec["gate_up"], spec["down"]), O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
        assert_close_bf16(to_np(ops.gateup_swiglu(to_dev(x, dev), Wgu)), ref["h"], f"h M={M}", ulps=8)
        hg = ops.gateup_swiglu(to_dev(x, dev), Wgu, gates=torch.from_numpy(g_ref).to(dev))
        assert_close_bf16(to_np(hg), refg["h"], f"gated h M={M}", ulps=8)


@pytest.mark.parametrize("d_model,rows", [(4096, (5, 8, 9, 16, 24, 32, 33, 64)), (5120, (5, 16, 32, 40, 64)), (8192, (3, 5, 8, 9, 16, 50))])
def test_gate_up_of_wide_models_at_decode_batches(dev, d_model, rows):
    """gate_up + SwiGLU for d_model 4096 / 5120 / 8192 at 3..64 rows: a 16-token tile of all K leaves no room for the
    part-split form's partial sums (or does not fit at all), so one 8- or 4-token tile of all K runs where the rows fit
    one, and K-segmented 16-token tiles (8 waves, one gate/up unit each) beyond.  Plain, gated, and the plain gate_up
    product (which takes several narrow tiles)."""
    d_ff, ncl = 16 * 24, 24
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=77, zipf_s=1.2)
    Wgu = synth.to_pack(spec["gate_up"], dev)
    for M in rows:
        x = synth.synth_x(M, d_model, 78 + M)
        g_ref = O.remoe_gates(synth.synth_logits(M, ncl, 79), 9)[0]
        ref, refg = O.swiglu_mlp(x, spec["gate_up"], spec["down"]), O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
        xd = to_dev(x, dev)
        assert_close_bf16(to_np(ops.gateup_swiglu(xd, Wgu)), ref["h"], f"h d_model={d_model} M={M}", ulps=8)
        hg = ops.gateup_swiglu(xd, Wgu, gates=torch.from_numpy(g_ref).to(dev))
        assert_close_bf16(to_np(hg), refg["h"], f"gated h d_model={d_model} M={M}", ulps=8)
        assert_close_bf16(to_np(ops.spmm(xd, Wgu)), oracle_spmm(x, spec["gate_up"]), f"gu d_model={d_model} M={M}", ulps=8)


@pytest.mark.parametrize("Cb,rows", [(688, (1, 4, 5, 8, 9, 16, 40)), (1024, (1, 3, 5, 8, 9)), (864, (2, 7, 8, 33))])
def test_down_of_wide_models_at_decode_batches(dev, Cb, rows):
    """`down` with 11008 / 16384 / 13824 input features (5, 7 and 6 K segments): the waves of a row unit share its parts
    also when their count divides by none of 4, 3, 2, and 5..8 rows run two 4-token tiles of all K; beyond that the
    K-segmented 16-token tiles.  Plain and with the routed input mask."""
    m = synth.synth_matrix(16 * 20, 16 * Cb, 0.25, seed=88, zipf_s=1.2)
    W = synth.to_pack(m, dev)
    assert W.nseg == {688: 5, 1024: 7, 864: 6}[Cb]
    ncl = Cb
    for M in rows:
        x = synth.synth_x(M, 16 * Cb, 89 + M)
        assert_close_bf16(to_np(ops.spmm(to_dev(x, dev), W)), oracle_spmm(x, m), f"Cb={Cb} M={M}", ulps=8)
        act = O.remoe_gates(synth.synth_logits(M, ncl, 90), ncl // 4)[1]
        got = ops.spmm(to_dev(x, dev), W, active=torch.from_numpy(act.astype(np.uint8)).to(dev))
        assert_close_bf16(to_np(got), oracle_spmm(x * np.repeat(act, 16, axis=1), m), f"masked Cb={Cb} M={M}", ulps=8)


@pytest.mark.parametrize("M", [65, 100, 128, 129])
def test_plain_product_over_k_segments_at_65_to_128_rows(dev, M):
    """65..128 rows of a matrix with several K segments run 8-token tiles of all K (a row's parts on different waves);
    one more row goes to the 32-token tiles: same product, plain and with the routed input mask, ragged rows."""
    d_ff, ncl = 16 * 352, 352
    m = synth.synth_matrix(16 * 40, d_ff, 0.25, seed=66, zipf_s=1.2)
    W = synth.to_pack(m, dev)
    assert W.nseg > 1
    x = synth.synth_x(M, d_ff, 67)
    assert_close_bf16(to_np(ops.spmm(to_dev(x, dev), W)), oracle_spmm(x, m), f"M={M}", ulps=8)
    act = O.remoe_gates(synth.synth_logits(M, ncl, 68), 88)[1]
    xm = x * np.repeat(act, d_ff // ncl, axis=1)
    got = ops.spmm(to_dev(x, dev), W, active=torch.from_numpy(act.astype(np.uint8)).to(dev))
    assert_close_bf16(to_np(got), oracle_spmm(xm, m), f"masked M={M}", ulps=8)


@pytest.mark.parametrize("max_blocks", [3, 8])
def test_decode_split_rows_partials(dev, max_blocks):
    spec = synth.synth_mlp(512, 16 * 90, 0.3, seed=60, zipf_s=1.2)
    x = synth.synth_x(5, 512, 61)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    h = ops.gemv(to_dev(x, dev), Wgu, swiglu_out=True, max_blocks=max_blocks)
    assert_close_bf16(to_np(h), ref["h"], "h", ulps=4)
    y = ops.gemv(h, Wdn, max_blocks=max_blocks)
    assert_close_bf16(to_np(y), ref["y"], "y", ulps=8)
    h1 = ops.gemv(to_dev(x, dev), Wgu, swiglu_out=True)
    assert_close_bf16(to_np(h), to_np(h1), "split vs whole", ulps=2)


@pytest.mark.parametrize("B", [1, 3])
def test_decode_routed(dev, B):
    d_model, d_ff, ncl, k = 512, 16 * 64, 64, 16
    spec = synth.synth_mlp(d_model, d_ff, 0.3, seed=70)
    x = synth.synth_x(B, d_model, 71)
    g_ref, _ = O.remoe_gates(synth.synth_logits(B, ncl, 72), k)
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=g_ref)
    gates = torch.from_numpy(g_ref).to(dev)
    mlp = synth.mlp_module(spec, dev)
    y = mlp(to_dev(x, dev), gates=gates)
    assert_close_bf16(to_np(y), ref["y"], "routed decode", ulps=8)
    dec = mortar_amd.MortarDecodeMLP(mlp)
    xr = O.rmsnorm(x)
    ref2 = O.swiglu_mlp(xr, spec["gate_up"], spec["down"], gates=g_ref)
    y2 = dec(to_dev(x, dev).reshape(B, 1, d_model), gates=gates)
    assert tuple(y2.shape) == (B, 1, d_model)
    assert_close_bf16(to_np(y2).reshape(B, d_model), ref2["y"], "engine mlp_fn", ulps=8)


def test_mortar_gemv_reference_signature(dev):
    spec = synth.synth_mlp(256, 512, 0.5, seed=80)
    mlp = synth.mlp_module(spec, dev)
    pk = mortar_amd.mortar_pack_strips(mlp.gate_up._cms)
    x = synth.synth_x(2, 256, 81)
    h = mortar_amd.mortar_gemv(torch.from_numpy(x).to(dev), pk, swiglu_out=True)      # fp32 in -> fp32 out
    assert h.dtype == torch.float32
    ref = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    assert_close_bf16(h.cpu().numpy(), ref["h"], "h", ulps=4)
    hb = mortar_amd.mortar_gemv(to_dev(x, dev), pk, swiglu_out=True)                   # bf16 in -> bf16 out
    assert hb.dtype == torch.bfloat16
    assert_close_bf16(to_np(hb), ref["h"], "h bf16", ulps=4)


def _gemv_f32_tolerance(ref):
    """fp32 sums of a few hundred exact products against float64: a few 1e-7 of the largest output (measured 2e-7)."""
    return 3e-6 * np.abs(ref).max()


@pytest.mark.parametrize("B", [1, 5, 16, 40])
@pytest.mark.parametrize("per_tensor", [False, True])
def test_mortar_gemv_fp32_arithmetic(dev, B, per_tensor):
    """mortar_gemv with fp32 activations against the oracle's decode form (exact +-x / 0 products, fp32 scale after the
    block sum, float64 sums): gate_up with SwiGLU (+ gates, row flags), then down, plain and with swiglu_x, with column
    flags and with rows split into partial slots."""
    d_model, d_ff, ncl = 512, 16 * 88, 22
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=95, zipf_s=1.2)
    if per_tensor:
        spec["gate_up"]["scales"] = spec["gate_up"]["scales"][:1] * 1.2345          # fp32 values that bf16 cannot hold
        spec["down"]["scales"] = spec["down"]["scales"][:1] * 0.987
    gu_m, dn_m = spec["gate_up"], spec["down"]
    assert not np.array_equal(O.bf16_round(gu_m["scales"]), gu_m["scales"])
    Wgu, Wdn = synth.to_pack(gu_m, dev), synth.to_pack(dn_m, dev)
    rng = np.random.default_rng(96 + B)
    x = rng.standard_normal((B, d_model)).astype(np.float32) * np.float32(1.37)          # full fp32 mantissas
    xt = torch.from_numpy(x).to(dev)
    gu = O.mortar_gemv(x, gu_m["codes"], gu_m["scales"], gu_m["col_idx"], gu_m["offsets"]).astype(np.float64)
    got_gu = ops.gemv_f32(xt, Wgu).cpu().numpy()
    assert np.abs(got_gu - gu).max() <= _gemv_f32_tolerance(gu)
    assert np.abs(ops.gemv_f32(xt, Wgu, max_blocks=3).cpu().numpy() - gu).max() <= _gemv_f32_tolerance(gu)   # partial slots
    # exactness beyond bf16: a bf16-rounded input gives a visibly different answer
    gu_b = O.mortar_gemv(O.bf16_round(x), gu_m["codes"], gu_m["scales"], gu_m["col_idx"], gu_m["offsets"])
    assert np.abs(gu_b - gu).max() > 100 * _gemv_f32_tolerance(gu)
    g, u = gu[:, :d_ff], gu[:, d_ff:]
    h_ref = g / (1.0 + np.exp(-g)) * u
    h = ops.gemv_f32(xt, Wgu, swiglu_out=True)
    assert h.dtype == torch.float32 and np.abs(h.cpu().numpy() - h_ref).max() <= _gemv_f32_tolerance(h_ref)
    # gates + row flags (route_flags): gated SwiGLU, inactive clusters exactly zero
    lg = torch.from_numpy(synth.synth_logits(B, ncl, 97)).to(dev)
    gates, active = ops.remoe_gates(lg, 6)
    ract, cact = ops.route_flags(gates, d_ff)
    hg_ref = (h_ref.reshape(B, ncl, -1) * gates.cpu().numpy().astype(np.float64)[:, :, None]).reshape(B, d_ff)
    hg = mortar_amd.mortar_gemv(xt, Wgu, swiglu_out=True, row_act=ract, gates=gates, cluster_size=d_ff // ncl)
    assert np.abs(hg.cpu().numpy() - hg_ref).max() <= _gemv_f32_tolerance(h_ref)
    off = np.repeat(~active.cpu().numpy().astype(bool), d_ff // ncl, axis=1)
    assert (hg.cpu().numpy()[off] == 0).all()
    # down: plain on h, with column flags on the gated h, and in the swiglu_x form on the raw gate_up output
    y_ref = O.mortar_gemv(h.cpu().numpy(), dn_m["codes"], dn_m["scales"], dn_m["col_idx"], dn_m["offsets"]).astype(np.float64)
    y = mortar_amd.mortar_gemv(h, Wdn)
    assert np.abs(y.cpu().numpy() - y_ref).max() <= _gemv_f32_tolerance(y_ref)
    yg_ref = O.mortar_gemv(hg.cpu().numpy(), dn_m["codes"], dn_m["scales"], dn_m["col_idx"], dn_m["offsets"])
    yg = mortar_amd.mortar_gemv(hg, Wdn, col_act=cact)
    assert np.abs(yg.cpu().numpy() - yg_ref).max() <= _gemv_f32_tolerance(yg_ref)
    y2 = mortar_amd.mortar_gemv(torch.from_numpy(got_gu).to(dev), Wdn, swiglu_x=True)
    assert np.abs(y2.cpu().numpy() - y_ref).max() <= 4 * _gemv_f32_tolerance(y_ref)


@pytest.mark.parametrize("B", [1, 3, 16, 22, 64])
def test_mortar_gemv_fp32_one_scale_runs_on_the_spmm_kernels(dev, B):
    """One scale per matrix and no flags: the fp32 product runs as 3 * B bf16 term rows through the SpMM kernels (one
    4-token tile, 16-token tiles, the 32-token prefill tiles at 3 * 64 rows, one and several K segments).  Checked against
    the oracle's float64 sums and against the work-list kernel (forced with an explicit split), incl. gates without
    flags and the swiglu_x form."""
    d_model, d_ff, ncl = 512, 16 * 200, 25
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=195, zipf_s=1.2)
    spec["gate_up"]["scales"] = spec["gate_up"]["scales"][:1] * 1.2345               # fp32 values that bf16 cannot hold
    spec["down"]["scales"] = spec["down"]["scales"][:1] * 0.987
    gu_m, dn_m = spec["gate_up"], spec["down"]
    Wgu, Wdn = synth.to_pack(gu_m, dev), synth.to_pack(dn_m, dev)
    assert Wdn.nseg > 1 and Wgu.scales_f32.numel() == 1
    rng = np.random.default_rng(196 + B)
    x = rng.standard_normal((B, d_model)).astype(np.float32) * np.float32(1.37)
    xt = torch.from_numpy(x).to(dev)
    gu = O.mortar_gemv(x, gu_m["codes"], gu_m["scales"], gu_m["col_idx"], gu_m["offsets"]).astype(np.float64)
    fast, slow = ops.gemv_f32(xt, Wgu).cpu().numpy(), ops.gemv_f32(xt, Wgu, max_blocks=1 << 20).cpu().numpy()
    assert np.abs(fast - gu).max() <= _gemv_f32_tolerance(gu) and np.abs(slow - gu).max() <= _gemv_f32_tolerance(gu)
    # a strided fp32 view (rows of a wider buffer, not 16-byte aligned) gives the same values
    wide = torch.zeros(B, d_model + 3, device=dev); wide[:, 1:d_model + 1] = xt
    assert np.array_equal(ops.gemv_f32(wide[:, 1:d_model + 1], Wgu).cpu().numpy(), fast)
    g, u = gu[:, :d_ff], gu[:, d_ff:]
    h_ref = g / (1.0 + np.exp(-g)) * u
    gates = ops.remoe_gates(torch.from_numpy(synth.synth_logits(B, ncl, 197)).to(dev), 7)[0]
    hg_ref = (h_ref.reshape(B, ncl, -1) * gates.cpu().numpy().astype(np.float64)[:, :, None]).reshape(B, d_ff)
    hg = ops.gemv_f32(xt, Wgu, swiglu_out=True, gates=gates)
    assert np.abs(hg.cpu().numpy() - hg_ref).max() <= _gemv_f32_tolerance(h_ref)
    h = ops.gemv_f32(xt, Wgu, swiglu_out=True)
    assert np.abs(h.cpu().numpy() - h_ref).max() <= _gemv_f32_tolerance(h_ref)
    y_ref = O.mortar_gemv(h.cpu().numpy(), dn_m["codes"], dn_m["scales"], dn_m["col_idx"], dn_m["offsets"]).astype(np.float64)
    for y in (ops.gemv_f32(h, Wdn), ops.gemv_f32(h, Wdn, max_blocks=1 << 20)):
        assert np.abs(y.cpu().numpy() - y_ref).max() <= _gemv_f32_tolerance(y_ref)
    y2 = ops.gemv_f32(torch.from_numpy(fast).to(dev), Wdn, swiglu_x=True)
    assert np.abs(y2.cpu().numpy() - y_ref).max() <= 4 * _gemv_f32_tolerance(y_ref)
    # flags without gates, both forms (SpMM kernels and work list), applied per stream as the reference's kernel does:
    # stream b's sum of row r is zero when row_act[b, r] == 0 (gate rows and up rows have flags of their own), and input
    # block-column c contributes nothing to stream b when col_act[b, c] == 0
    ract_np = (rng.random((B, 2 * d_ff // 16)) < 0.5).astype(np.int32)
    ract_np[:, 3] = 0; ract_np[:, 5] = 1                                           # a unit off / on for every stream
    cact_np = (rng.random((B, d_ff // 16)) < 0.5).astype(np.int32)
    ract, cact = torch.from_numpy(ract_np).to(dev), torch.from_numpy(cact_np).to(dev)
    gu_f = O.mortar_gemv(x, gu_m["codes"], gu_m["scales"], gu_m["col_idx"], gu_m["offsets"], row_act=ract_np).astype(np.float64)
    gf, uf = gu_f[:, :d_ff], gu_f[:, d_ff:]
    want = gf / (1.0 + np.exp(-gf)) * uf
    for kw in ({}, {"max_blocks": 1 << 20}, {"max_blocks": 8}):
        got = ops.gemv_f32(xt, Wgu, swiglu_out=True, row_act=ract, **kw).cpu().numpy()
        assert np.abs(got - want).max() <= _gemv_f32_tolerance(h_ref), kw
        assert (got[np.repeat(ract_np[:, :d_ff // 16] == 0, 16, axis=1)] == 0).all()
        got = ops.gemv_f32(xt, Wgu, row_act=ract, **kw).cpu().numpy()               # plain product, a flag per output row
        assert np.abs(got - gu_f).max() <= _gemv_f32_tolerance(gu), kw
    ym_ref = O.mortar_gemv(h.cpu().numpy(), dn_m["codes"], dn_m["scales"], dn_m["col_idx"], dn_m["offsets"], col_act=cact_np).astype(np.float64)
    for kw in ({}, {"max_blocks": 1 << 20}, {"max_blocks": 8}):
        got = ops.gemv_f32(h, Wdn, col_act=cact, **kw).cpu().numpy()
        assert np.abs(got - ym_ref).max() <= _gemv_f32_tolerance(y_ref), kw


@pytest.mark.parametrize("B,n,f32", [(1, 4, True), (3, 4, False), (16, 2, True), (40, 4, False), (5, 1, True), (7, 3, False)])
def test_down_with_hc_post_epilogue(dev, B, n, f32):
    """`down` with the hyper-connection POST write in its epilogue against the oracle (y rounded to bf16, then the
    float64 combination), for fp32 and bf16 carriers, with and without the inject term and the routed input mask."""
    d_model, d_ff = 512, 16 * 96
    m = synth.synth_matrix(d_model, d_ff, 0.25, seed=90)
    W = synth.to_pack(m, dev)
    rng = np.random.default_rng(91 + B)
    x = synth.synth_x(B, d_ff, 92)
    dt = torch.float32 if f32 else torch.bfloat16
    rnd = (lambda a: a.astype(np.float32)) if f32 else (lambda a: O.bf16_round(a.astype(np.float32)))
    h = rnd(rng.standard_normal((B, n, d_model)))
    term = rnd(rng.standard_normal((B, d_model)))
    hres = (rng.standard_normal((B, n, n)) * 0.5).astype(np.float32)
    hpost = rng.standard_normal((B, n)).astype(np.float32)
    T = lambda a, d=None: torch.from_numpy(a).to(dev).to(d) if d is not None else torch.from_numpy(a).to(dev)
    y = oracle_spmm(x, m)                                                   # bf16-rounded, as the unfused path stores it
    tol = dict(rtol=2e-6, atol=2e-6) if f32 else dict(rtol=2.0 ** -7, atol=1e-2)
    for use_term in (False, True):
        ref = O.hc_post(hres, hpost, h, y, term if use_term else None)
        got = ops.spmm_hc_post(to_dev(x, dev), W, T(h, dt), T(hres), T(hpost), T(term, dt) if use_term else None)
        assert got.dtype == dt and tuple(got.shape) == (B, n, d_model)
        yk = to_np(ops.spmm(to_dev(x, dev), W))                             # the kernel's own y: same bits go into the POST
        ref_k = O.hc_post(hres, hpost, h, yk, term if use_term else None)
        np.testing.assert_allclose(got.float().cpu().numpy(), ref_k, **tol)
        assert np.abs(got.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()
    # identity mixing and hpost = 0 returns the carrier bit for bit; hres = 0, hpost = 1 returns y in every stream
    eye = torch.eye(n, device=dev).expand(B, n, n).contiguous()
    out = ops.spmm_hc_post(to_dev(x, dev), W, T(h, dt), eye, torch.zeros(B, n, device=dev))
    assert torch.equal(out, T(h, dt))
    out = ops.spmm_hc_post(to_dev(x, dev), W, T(h, dt), torch.zeros(B, n, n, device=dev), torch.ones(B, n, device=dev))
    assert torch.equal(out.float(), ops.spmm(to_dev(x, dev), W).float()[:, None, :].expand(B, n, d_model))
    # routed: inactive input clusters read as zero, as in the masked product
    act = torch.from_numpy((rng.random((B, 16)) < 0.5).astype(np.uint8)).to(dev)
    ym = ops.spmm(to_dev(x, dev), W, active=act)
    out = ops.spmm_hc_post(to_dev(x, dev), W, T(h, dt), torch.zeros(B, n, n, device=dev), torch.ones(B, n, device=dev), active=act)
    assert torch.equal(out.float(), ym.float()[:, None, :].expand(B, n, d_model))
    with pytest.raises(ValueError, match="decode batches"):
        ops.spmm_hc_post(to_dev(synth.synth_x(65, d_ff, 1), dev), W, torch.zeros(65, n, d_model, device=dev),
                         torch.zeros(65, n, n, device=dev), torch.zeros(65, n, device=dev))


def test_rmsnorm(dev):
    x = O.bf16_round(synth.synth_x(37, 2048, 90) * 3)
    w = synth.synth_x(1, 2048, 91)[0]
    y = ops.rmsnorm(to_dev(x, dev), to_dev(w, dev))
    assert_close_bf16(to_np(y), O.rmsnorm(x, w), "rmsnorm", ulps=2)
    y = ops.rmsnorm(to_dev(x, dev).reshape(37, 1, 2048))
    assert_close_bf16(to_np(y).reshape(37, 2048), O.rmsnorm(x), "rmsnorm unit weight", ulps=2)


@pytest.mark.parametrize("d_model,M", [(256, 1), (256, 3), (256, 16), (256, 40), (256, 200), (2048, 1), (2048, 5),
                                       (2048, 200), (16 * 47, 130)])
def test_norm_fused_into_gate_up(dev, d_model, M):
    """RMSNorm applied while gate_up stages x gives the bits of rmsnorm() followed by gateup_swiglu(), for the decode
    tiles (part-split and small workgroups), the 64- and 32-token prefill tiles, with and without weight, gated and
    routed; and agrees with the oracle."""
    d_ff = 16 * 24
    spec = synth.synth_mlp(d_model, d_ff, 0.25, seed=60, zipf_s=1.2)
    x = O.bf16_round(synth.synth_x(M, d_model, 61) * 2.5)
    w = O.bf16_round(1.0 + 0.1 * synth.synth_x(1, d_model, 62)[0])
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    assert ops.norm_fusable(Wgu)
    xd, wd = to_dev(x, dev), to_dev(w, dev)
    gates, active = ops.remoe_gates(torch.from_numpy(synth.synth_logits(M, d_ff // 16, 63)).to(dev), 6)
    for nw, eps in ((wd, 1e-6), (None, 1e-5)):
        xn = ops.rmsnorm(xd, nw, eps)
        assert torch.equal(ops.gateup_swiglu(xd, Wgu, norm=(nw, eps)), ops.gateup_swiglu(xn, Wgu))
        assert torch.equal(ops.gateup_swiglu(xd, Wgu, gates=gates, norm=(nw, eps)), ops.gateup_swiglu(xn, Wgu, gates=gates))
        tile = ops.route_tile(Wgu, M)
        route = ops.remoe_route(active, tile)
        a, b = torch.zeros((M, d_ff), dtype=torch.bfloat16, device=dev), torch.zeros((M, d_ff), dtype=torch.bfloat16, device=dev)
        ops.gateup_swiglu(xd, Wgu, gates=gates, route=route, norm=(nw, eps), out=a)
        ops.gateup_swiglu(xn, Wgu, gates=gates, route=route, out=b)
        assert torch.equal(a, b)
    ref = O.swiglu_mlp(O.rmsnorm(x, w), spec["gate_up"], spec["down"])
    h = ops.gateup_swiglu(xd, Wgu, norm=(wd, 1e-6))
    assert_close_bf16(to_np(h), ref["h"], "h of normalised x", ulps=8)
    mlp = synth.mlp_module(spec, dev)
    assert torch.equal(mlp(xd, norm=(wd, 1e-6)), mlp(ops.rmsnorm(xd, wd, 1e-6)))


def test_norm_fusion_limits(dev):
    """Matrices too wide for the fused norm are refused by the C-ABI; the module falls back to a separate launch."""
    spec = synth.synth_mlp(16 * 130, 16 * 8, 0.25, seed=64)
    Wgu = synth.to_pack(spec["gate_up"], dev)
    xd = to_dev(synth.synth_x(20, 16 * 130, 65), dev)
    assert not ops.norm_fusable(Wgu)
    with pytest.raises(ValueError, match="fused RMSNorm"):
        ops.gateup_swiglu(xd, Wgu, norm=(None, 1e-6))
    mlp = synth.mlp_module(spec, dev)
    assert torch.equal(mlp(xd, norm=(None, 1e-6)), mlp(ops.rmsnorm(xd, None, 1e-6)))


def test_looped_core_stack_small(dev):
    """benchmark config 4 call pattern at reduced size: shared blocks x iterations, RMS-normalised input, Zipf rows."""
    d_model, d_ff, M = 256, 16 * 44, 150
    specs = [synth.synth_mlp(d_model, d_ff, 0.25, seed=200 + i, zipf_s=1.2) for i in range(2)]
    x = synth.synth_x(M, d_model, 210)
    ref = x
    for t in range(3):
        for s in specs:
            ref = O.swiglu_mlp(O.rmsnorm(ref), s["gate_up"], s["down"])["y"]
    mlps = [synth.mlp_module(s, dev) for s in specs]
    y = mortar_amd.looped_core_forward(mlps, to_dev(x, dev), 3)
    assert_close_bf16(to_np(y), ref, "looped stack", ulps=64, max_rel=2e-2)


def test_looped_core_stack_full_size(dev):
    """benchmark config 4 at its own size: 8 shared blocks x 6 iterations, d_model 2048 / d_ff 5632, 4096 tokens,
    Zipf(1.2) row lengths clipped to 5-60 %, RMSNorm (with a weight) folded into every gate_up launch.
    Every one of the 48 MLP calls is checked on sampled rows against the oracle fed the HIP input of THAT call,
    so the error of earlier calls does not compound into the comparison; the final output is checked for
    finiteness and for the row RMS the oracle's last call predicts."""
    d_model, d_ff, M, n_blocks, n_iters = 2048, 5632, 4096, 8, 6
    specs = [synth.synth_mlp(d_model, d_ff, 0.25, seed=400 + i, zipf_s=1.2) for i in range(n_blocks)]
    for s in specs:                                            # the rows really are uneven
        cnt = np.diff(s["gate_up"]["offsets"])
        assert cnt.min() <= 0.06 * 128 + 1 and cnt.max() >= 0.55 * 128
    rng = np.random.default_rng(410)
    norm_w = [O.bf16_round(rng.uniform(0.5, 1.5, d_model).astype(np.float32)) for _ in range(n_blocks)]
    mlps = [synth.mlp_module(s, dev) for s in specs]
    assert all(ops.norm_fusable(m.gate_up._cms.mortar_pack()) for m in mlps)
    rows = np.array([0, 31, 32, 1000, 2047, 2048, 3333, 4095])
    rows_t = torch.from_numpy(rows).to(dev)
    seen = []
    def observer(t, i, x_in, x_out):
        seen.append((t, i, x_in[rows_t].float().cpu().numpy(), x_out[rows_t].float().cpu().numpy()))
    x = synth.synth_x(M, d_model, 411)
    y = mortar_amd.looped_core_forward(mlps, to_dev(x, dev), n_iters, norm_weights=[to_dev(w, dev) for w in norm_w],
                                       observer=observer)
    assert len(seen) == n_blocks * n_iters and [(t, i) for t, i, _, _ in seen] == \
        [(t, i) for t in range(n_iters) for i in range(n_blocks)]
    assert np.array_equal(seen[0][2], x[rows])
    for k, (t, i, xin, yout) in enumerate(seen):
        ref = O.swiglu_mlp(O.rmsnorm(xin, norm_w[i], 1e-6), specs[i]["gate_up"], specs[i]["down"])["y"]
        assert_close_bf16(yout, ref, f"iteration {t} block {i}", ulps=8, max_rel=1e-2)
        if k + 1 < len(seen):
            assert np.array_equal(seen[k + 1][2], yout)                   # the next call reads this output unchanged
    yn = to_np(y)
    assert np.isfinite(yn).all() and np.array_equal(yn[rows], seen[-1][3])
    rms = np.sqrt((yn.astype(np.float64) ** 2).mean(1))
    assert rms.min() > 0 and rms.max() / np.median(rms) < 10 and rms.min() / np.median(rms) > 0.1


def test_known_answers_on_the_device(dev):
    """Hand-written cases of the three rules a loose test would let slip: the strict threshold of the ternary rule,
    the place of eps in the RMSNorm, and the lo side of a straddling block in route_flags."""
    # RMSNorm: x = (3, 4) * 2^-8 (bf16-exact) repeated: mean(x^2) = 12.5 * 2^-16, eps = 2^-16 -> y = x * 2^8 / sqrt(13.5)
    x = np.tile(np.array([3.0, 4.0], np.float32) * 2.0 ** -8, (3, 64))
    y = to_np(ops.rmsnorm(to_dev(x, dev), None, 2.0 ** -16))
    want = O.bf16_round(np.tile(np.array([3.0, 4.0]) / np.sqrt(13.5), (3, 64)).astype(np.float32))
    assert np.array_equal(y, want), (y[0, :2], want[0, :2])              # eps outside the root gives 0.664 / 0.886
    assert np.array_equal(y, O.rmsnorm(x, None, 2.0 ** -16))
    # the fused form (norm applied while gate_up stages x) sees the same eps
    spec = synth.synth_mlp(128, 64, 0.5, seed=77)
    Wgu = synth.to_pack(spec["gate_up"], dev)
    xd = to_dev(x, dev)
    assert torch.equal(ops.gateup_swiglu(xd, Wgu, norm=(None, 2.0 ** -16)), ops.gateup_swiglu(to_dev(want, dev), Wgu))
    # route_flags, clusters of 8 (a 16-wide block spans lo = 2r and hi = 2r + 1): lo side alone, hi side alone
    g = torch.zeros((3, 16), device=dev); g[0, 2] = 1.0; g[1, 3] = 0.5; g[2, 14] = 0.25
    ract, cact = ops.route_flags(g, 128)
    assert cact.cpu().tolist() == [[0, 1, 0, 0, 0, 0, 0, 0], [0, 1, 0, 0, 0, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 1]]
    assert ract.cpu().tolist() == [c + c for c in cact.cpu().tolist()]
    gz = torch.zeros((1, 16), device=dev); gz[0, 2] = -1.0; gz[0, 5] = float("nan")
    assert int(ops.route_flags(gz, 128)[1].sum()) == 0


# ---------------------------------------------------------------------------------------------- full size, by properties

def test_full_size_properties(dev):
    """benchmark config 3 shapes (d_model 2048, d_ff 5632, 4096 tokens): size-independent checks.
    (1) rows sampled from the prefill output equal the oracle on those rows; (2) prefill and decode kernels
    agree on the same rows; (3) linearity in a power-of-two scale is exact."""
    spec = synth.synth_mlp(2048, 5632, 0.25, seed=300)
    Wgu, Wdn = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    x = synth.synth_x(4096, 2048, 301)
    xd = to_dev(x, dev)
    h = ops.gateup_swiglu(xd, Wgu)
    y = ops.spmm(h, Wdn)
    rows = np.array([0, 1, 127, 128, 2047, 4095, 1234, 3071])
    ref = O.swiglu_mlp(x[rows], spec["gate_up"], spec["down"])
    assert_close_bf16(to_np(h)[rows], ref["h"], "h rows", ulps=4)
    assert_close_bf16(to_np(y)[rows], ref["y"], "y rows", ulps=8)
    hd = ops.gemv(xd[rows], Wgu, swiglu_out=True)
    assert_close_bf16(to_np(hd), to_np(h)[rows], "decode vs prefill h", ulps=2)
    gu = ops.spmm(xd, Wgu)
    gu4 = ops.spmm(xd * 4, Wgu)
    assert torch.equal(gu4.float(), gu.float() * 4)
    # routed, full size: selection bit-exact and sampled rows against the oracle
    lg = synth.synth_logits(4096, 352, 302)
    g_ref, a_ref = O.remoe_gates(lg, 88)
    gates, active = ops.remoe_gates(torch.from_numpy(lg).to(dev), 88)
    assert np.array_equal(active.cpu().numpy().astype(bool), a_ref)
    cnt, lst = ops.remoe_route(active, ops.route_tile(Wgu, 4096))
    assert int(cnt.sum()) == int(a_ref.sum())
    hr = ops.gateup_swiglu(xd, Wgu, gates=gates, route=(cnt, lst))
    yr = ops.spmm(hr, Wdn, active=active)
    refr = O.swiglu_mlp(x[rows], spec["gate_up"], spec["down"], gates=g_ref[rows])
    assert_close_bf16(to_np(yr)[rows], refr["y"], "routed y rows", ulps=8)


# ---------------------------------------------------------------------------------------------- error behaviour

def test_argument_errors_are_raised_before_launch(dev):
    """Host-side checks of the C-ABI surface: every bad call raises (ValueError for arguments / limits) and
    nothing is launched."""
    m = synth.synth_matrix(16 * 4, 16 * 8, 0.5, seed=1)
    W = synth.to_pack(m, dev)
    x = to_dev(synth.synth_x(8, 128, 2), dev)
    with pytest.raises(ValueError, match="features"):
        ops.spmm(x[:, :64], W)
    with pytest.raises(TypeError):
        ops.spmm(x.float(), W)
    with pytest.raises(RuntimeError, match="ROCm device"):
        ops.spmm(x.cpu(), W)
    with pytest.raises(ValueError, match="odd number of block-rows"):
        ops.gateup_swiglu(x, synth.to_pack(synth.synth_matrix(16 * 3, 16 * 8, 0.5, seed=2), dev))
    with pytest.raises(ValueError, match="multiple of 4"):                       # d_ff / n_clusters = 32 / 16 = 2
        ops.gateup_swiglu(x, W, gates=torch.ones((8, 16), device=dev))
    with pytest.raises(ValueError, match="tile must be"):
        ops.remoe_route(torch.ones((8, 4), dtype=torch.uint8, device=dev), 24)
    wide = synth.to_pack(synth.synth_matrix(16 * 4, 16 * 400, 0.1, seed=3), dev)  # K too wide for routed skipping
    assert ops.route_tile(wide, 4096) == 0 and ops.route_tile(wide, 2) == 4
    assert ops.spmm(x[:0], W).shape == (0, 64)                                    # empty batch: no launch, empty result
    y = ops.spmm(x, W)                                                            # and the good call still works
    assert_close_bf16(to_np(y), oracle_spmm(to_np(x), m), "after errors")


def test_raw_c_abi_refuses_bad_calls_of_the_newer_entry_points(dev):
    """mortar_mlp_bf16, mortar_dds_values_bf16 and mortar_router_tail_f32 called through ctypes with bad arguments return a
    negative code and a message, launch nothing, and leave the outputs untouched."""
    import ctypes as C
    from mortar_amd import _lib
    from mortar_amd.pack import BcsrTopology
    L = _lib.lib()
    err = lambda: C.c_char_p(L.mortar_last_error()).value.decode()
    spec = synth.synth_mlp(256, 640, 0.25, seed=7)
    G, D = synth.to_pack(spec["gate_up"], dev), synth.to_pack(spec["down"], dev)
    x = to_dev(synth.synth_x(40, 256, 8), dev)
    y = torch.full((40, 256), 7.0, dtype=torch.bfloat16, device=dev)
    ws = torch.zeros(ops.mlp_hidden_bytes(40, 640), dtype=torch.uint8, device=dev)
    p = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    call = lambda Wg, Wd, hidden, phase: L.mortar_mlp_bf16(Wg.ref, p(Wg.sched(2)), Wd.ref, p(Wd.sched(1)), p(x), 40, 256, 0, None, 0.0,
                                                             None, 0, hidden, p(y), 256, phase, st)
    assert call(G, D, None, 0) < 0 and "null" in err()
    assert call(D, G, p(ws), 0) < 0                                     # matrices swapped: shapes do not chain
    assert call(G, D, p(ws), 3) < 0 and "phase" in err()
    assert call(G, D, C.c_void_p(ws.data_ptr() + 2), 0) < 0 and "aligned" in err()
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())
    assert call(G, D, p(ws), 0) == 0                                    # and the good call runs
    torch.cuda.synchronize()
    assert_close_bf16(to_np(y), O.swiglu_mlp(to_np(x), spec["gate_up"], spec["down"])["y"], "mlp after refused calls", ulps=8)

    m = spec["down"]
    T = BcsrTopology(m["offsets"], m["col_idx"], m["shape"][0], m["shape"][1], dev)
    data = torch.zeros((T.nnz, 16, 16), dtype=torch.bfloat16, device=dev)
    h = to_dev(synth.synth_x(40, 640, 9), dev)
    y.fill_(7.0)
    dds = lambda xp, M, ldx: L.mortar_dds_values_bf16(p(T.row_ptr), p(T.col), None, p(data), T.Rb, T.Cb, T.nnz, xp, M, ldx, p(y), 256, st)
    assert dds(None, 40, 640) < 0 and dds(p(h), -1, 640) < 0 and dds(p(h), 40, 100) < 0
    assert dds(C.c_void_p(h.data_ptr() + 2), 40, 640) < 0
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())

    z = lambda *shape: torch.zeros(shape, device=dev)
    qv, g = z(8, 256), torch.full((8, 16), 7.0, device=dev)
    tail = lambda d, ldq, nsk, n, k: L.mortar_router_tail_f32(p(qv), 8, d, ldq, None, p(z(256)), p(z(256)), 1e-5, p(z(4, 128)), p(z(4, 128)), nsk, p(z(16)),
                                                               n, k, None, p(g), None, st)
    assert tail(250, 256, 4, 16, 4) < 0 and tail(256, 100, 4, 16, 4) < 0 and tail(256, 256, 0, 16, 4) < 0 and tail(256, 256, 4, 16, 0) < 0
    assert tail(256, 256, 40, 16, 4) < 0 and "product keys" in err()
    torch.cuda.synchronize()
    assert bool((g == 7.0).all())

