"""GPU parity of the device-side re-pack (ternarise + encode on the device) and of the W^T pack it fills for the
dX product, against the CPU oracle and the host packer.  Codes and layouts bit-exact; bf16 outputs to 1e-2."""
import numpy as np
import pytest
import torch

from mortar_amd import ops, synth
from mortar_amd.pack import MortarPack, decode_blocks
from oracle import mortar_oracle as O
from util import assert_close_bf16, to_dev, to_np

pytestmark = pytest.mark.gpu

ARRAYS = ("codes", "sdup", "codes_o", "sd_o", "codes4_o")


def _values(nnz, seed, dtype):
    rng = np.random.Generator(np.random.PCG64(seed))
    v = rng.standard_normal((nnz, 16, 16), dtype=np.float32) * rng.uniform(0.01, 0.1, (nnz, 1, 1)).astype(np.float32)
    v[rng.random((nnz, 16, 16)) < 0.05] = 0.0
    v[0, 0, :4] = [0.0, -0.0, 1e-30, -1e-30]
    t = torch.from_numpy(v).to(dtype)
    return t, t.float().numpy()


def _rule(w, s, thr):
    """The reference's rule with the scale given, in fp32 as torch computes it (deploy_quant.py:92-94)."""
    wn = w / np.float32(1.0) / s
    return (np.sign(wn) * (np.abs(wn) > np.float32(thr))).astype(np.int8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("per_block", [False, True])
@pytest.mark.parametrize("shape,seg", [((16 * 12, 16 * 30), None), ((16 * 6, 16 * 352), None)])
def test_requantize_equals_the_host_pack(dev, dtype, per_block, shape, seg):
    m = synth.synth_matrix(shape[0], shape[1], 0.25, seed=11, zipf_s=1.2)
    nnz = m["col_idx"].size
    vt, v = _values(nnz, 12, dtype)
    W = MortarPack(None, None, m["col_idx"], m["offsets"], shape[0], shape[1], dev)
    thr = 0.5
    s_dev = W.requantize(vt.to(dev), per_block=per_block, threshold=thr).cpu().numpy()
    # scale: the oracle's mean|w| (fp32 pairwise) against the device's (fp64 sum, rounded once): a few ulps apart at most
    qo, so = (O.ternary_quantize_per_block if per_block else O.ternary_quantize)(v, thr)
    np.testing.assert_allclose(s_dev, np.atleast_1d(so), rtol=4e-7, atol=0)
    # codes: exactly the rule under the device's own scale, and the oracle's codes except on the threshold itself
    s_full = s_dev[:, None, None] if per_block else s_dev[0]
    q = _rule(v, s_full, thr)
    got = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
    assert np.array_equal(got, q)
    differ = got != qo
    assert differ.mean() < 1e-5 and np.all(np.abs(np.abs(v / s_full)[differ] - thr) < 1e-5)
    # every device array equals what the host packer builds from the same codes and scales
    H = MortarPack(synth.flat_pack(q), s_dev if per_block else s_dev[:1], m["col_idx"], m["offsets"], shape[0], shape[1], dev)
    for name in ARRAYS:
        assert torch.equal(getattr(W, name), getattr(H, name)), name
    assert W.uniform_scale == H.uniform_scale and (W.uniform_scale != 0) == (not per_block)
    # and the product through it
    x = synth.synth_x(70, shape[1], seed=13)
    ref = O.bcsr_spmm(x, q, O.bf16_round(np.broadcast_to(s_dev, (nnz,)) if per_block else np.full(nnz, s_dev[0], np.float32)),
                      m["col_idx"], m["offsets"])
    assert_close_bf16(to_np(ops.spmm(to_dev(x, dev), W)), ref, "spmm after requantize")


def test_requantize_threshold_is_strict(dev):
    """Known answers at the cut (deploy_quant.py:94, strict >): values exactly on threshold * mean|w| get code 0."""
    m = dict(col_idx=np.array([0, 1], np.int16), offsets=np.array([0, 2], np.int32))
    W = MortarPack(None, None, m["col_idx"], m["offsets"], 16, 32, dev)
    for dtype in (torch.float32, torch.bfloat16):
        v = np.full((2, 16, 16), 2.0, np.float32)
        v[:, 0, :8] = 1.0; v[:, 1, :8] = -3.0                     # per block: mean|w| = (240*2 + 8 + 24) / 256 = 2 exactly
        v[1] *= -0.5                                              # second block: mean 1, the entries -0.5 on the cut
        vt = torch.from_numpy(v).to(dtype).to(dev)
        s = W.requantize(vt, per_block=True, threshold=0.5).cpu().numpy()
        assert s.tolist() == [2.0, 1.0]
        q = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
        assert (q[0, 0, :8] == 0).all() and (q[0, 1, :8] == -1).all() and (q[0, 2:] == 1).all() and (q[0, 0, 8:] == 1).all()
        assert (q[1, 0, :8] == 0).all() and (q[1, 1, :8] == 1).all() and (q[1, 2:] == -1).all()
        assert np.array_equal(q, O.ternary_quantize_per_block(v)[0])
        # per matrix: mean|w| = 1.5, cut at 0.75: |v| = 0.5 drops, 1.0 and above stay
        s = W.requantize(vt, per_block=False, threshold=0.5).cpu().numpy()
        assert s.tolist() == [1.5]
        q = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
        assert (q[0, 0, :8] == 1).all() and (q[1, 0, :8] == 0).all() and np.array_equal(q, O.ternary_quantize(v)[0])
    v = np.full((2, 16, 16), 4.0, np.float32); v[:, 0, :] = 2.0; v[:, 1, :] = 6.0          # mean|w| = 4 exactly
    s = W.requantize(torch.from_numpy(v).to(dev), per_block=False, threshold=0.5).cpu().numpy()
    q = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
    assert s.tolist() == [4.0] and (q[:, 0, :] == 0).all() and (q[:, 1:, :] == 1).all()


def test_requantize_given_scales_and_refresh(dev):
    """Given scales (one or per block), a second refresh with other values, and the asynchronous form."""
    m = synth.synth_matrix(16 * 8, 16 * 24, 0.3, seed=21)
    nnz = m["col_idx"].size
    W = MortarPack(None, None, m["col_idx"], m["offsets"], 16 * 8, 16 * 24, dev)
    for seed, scale in ((1, np.array([0.037], np.float32)), (2, np.linspace(0.01, 0.2, nnz).astype(np.float32))):
        vt, v = _values(nnz, seed, torch.bfloat16)
        s = W.requantize(vt.to(dev), scale=torch.from_numpy(scale), threshold=0.7, sync=False)
        assert np.array_equal(s.cpu().numpy(), scale) and W.uniform_scale == 0.0
        q = _rule(v, scale[:, None, None] if scale.size > 1 else scale[0], 0.7)
        H = MortarPack(synth.flat_pack(q), scale, m["col_idx"], m["offsets"], 16 * 8, 16 * 24, dev)
        for name in ARRAYS:
            assert torch.equal(getattr(W, name), getattr(H, name)), (seed, name)


def test_requantize_rejects_bad_input(dev):
    m = synth.synth_matrix(16 * 4, 16 * 8, 0.5, seed=3)
    nnz = m["col_idx"].size
    W = MortarPack(None, None, m["col_idx"], m["offsets"], 64, 128, dev)
    with pytest.raises(ValueError):
        W.requantize(torch.zeros(nnz, 16, 16, device=dev, dtype=torch.float16))
    with pytest.raises(ValueError):
        W.requantize(torch.zeros(nnz + 1, 16, 16, device=dev))
    with pytest.raises(ValueError):
        W.requantize(torch.zeros(nnz, 16, 16, device=dev), threshold=-1.0)
    with pytest.raises(ValueError):                      # scale far outside the bf16 window the kernels accept
        W.requantize(torch.ones(nnz, 16, 16, device=dev), scale=torch.tensor([1e35]))
    # all-zero values: scale clamps (1e-8 / 1e-6), every code is 0, products are 0
    W.requantize(torch.zeros(nnz, 16, 16, device=dev), per_block=True)
    assert int(W.codes.abs().sum()) == 0
    y = ops.spmm(torch.ones(5, 128, device=dev, dtype=torch.bfloat16), W)
    assert float(y.abs().max()) == 0.0


@pytest.mark.parametrize("per_block", [False, True])
@pytest.mark.parametrize("M", [3, 200])
@pytest.mark.parametrize("shape,density", [((16 * 20, 16 * 12), 0.3), ((16 * 3, 16 * 40), 0.1)])
def test_transposed_pack_gives_the_dx_product(dev, per_block, M, shape, density):
    """dX = dY @ W through the W^T pack (the reference's dds with the transposed metadata, transpose_b=False).  The
    second shape has block-columns without any block: those slices of dX are zero."""
    m = synth.synth_matrix(shape[0], shape[1], density, seed=31, zipf_s=1.2)
    nnz = m["col_idx"].size
    vt, v = _values(nnz, 32, torch.bfloat16)
    W = MortarPack(None, None, m["col_idx"], m["offsets"], shape[0], shape[1], dev)
    s = W.requantize(vt.to(dev), per_block=per_block).cpu().numpy()
    Wt = W.transposed()
    st = Wt.requantize(vt.to(dev), per_block=per_block, transpose=True).cpu().numpy()
    src = Wt.src_block.cpu().numpy()
    assert np.array_equal(st, s[src] if per_block else s)
    # W^T's blocks are W's blocks transposed, in the transposed order
    cw = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
    ct = decode_blocks(Wt.codes.cpu().numpy().view(np.uint32))
    assert np.array_equal(ct, cw[src].transpose(0, 2, 1))
    dense = O.to_dense(cw.astype(np.float32) * O.bf16_round(np.broadcast_to(s, (nnz,)))[:, None, None],
                       m["row_idx"], m["col_idx"], shape)
    dy = synth.synth_x(M, shape[0], seed=33)
    ref = O.bf16_round(dy).astype(np.float64) @ dense.astype(np.float64)
    assert_close_bf16(to_np(ops.spmm(to_dev(dy, dev), Wt)), ref.astype(np.float32), "dX")


def test_stk_dds_both_orientations(dev):
    """The operator signature with transpose_b=False (dX = dY @ W) next to the forward orientation, and a refresh
    after the data tensor changed in place."""
    import mortar_amd
    m = synth.synth_matrix(16 * 8, 16 * 6, 0.5, seed=41)
    t = lambda a: torch.from_numpy(a).to(dev)
    data = t(O.effective_blocks(m["codes"], m["scales"])).to(torch.bfloat16)
    dense = O.to_dense(data.float().cpu().numpy(), m["row_idx"], m["col_idx"], (128, 96)).astype(np.float64)
    z32, z16 = torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int16, device=dev)
    args = (t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32)
    x, dy = synth.synth_x(40, 96, seed=42), synth.synth_x(40, 128, seed=43)
    y = mortar_amd.stk_dds(to_dev(x, dev), data, *args, 96, 128, True)
    dx = mortar_amd.stk_dds(to_dev(dy, dev), data, *args, 128, 96, False)
    assert y.shape == (40, 128) and dx.shape == (40, 96) and dx.dtype == torch.bfloat16
    assert_close_bf16(to_np(y), (O.bf16_round(x) @ dense.T).astype(np.float32), "forward")
    assert_close_bf16(to_np(dx), (O.bf16_round(dy) @ dense).astype(np.float32), "dX")
    data.mul_(-2.0)                                     # same storage, new version: both packs must follow
    y2 = mortar_amd.stk_dds(to_dev(x, dev), data, *args, 96, 128, True)
    dx2 = mortar_amd.stk_dds(to_dev(dy, dev), data, *args, 128, 96, False)
    assert_close_bf16(to_np(y2), (-2.0 * (O.bf16_round(x) @ dense.T)).astype(np.float32), "forward refreshed")
    assert_close_bf16(to_np(dx2), (-2.0 * (O.bf16_round(dy) @ dense)).astype(np.float32), "dX refreshed")


# ---------------------------------------------------------------------------------------------- weight gradient

@pytest.mark.parametrize("shape,density,zipf,M", [((16 * 4, 16 * 6), 1.0, None, 32), ((16 * 20, 16 * 12), 0.3, 1.2, 1),
                                                   ((16 * 2, 16 * 1), 1.0, None, 33), ((16 * 3, 16 * 5), 0.6, None, 95),
                                                   ((16 * 1, 16 * 90), 1.0, None, 64), ((16 * 130, 16 * 2), 0.5, None, 40),
                                                   ((16 * 20, 16 * 12), 0.3, 1.2, 77), ((16 * 40, 16 * 30), 0.25, None, 600),
                                                   ((16 * 6, 16 * 352), 0.25, 1.2, 200), ((16 * 70, 16 * 16), 0.1, None, 4096)])
def test_sdd_weight_gradient(dev, shape, density, zipf, M):
    """dW on the topology against the oracle (one and several K segments, ragged token counts, split token ranges)."""
    m = synth.synth_matrix(shape[0], shape[1], density, seed=51, zipf_s=zipf)
    W = synth.to_pack(m, dev)
    a, b = synth.synth_x(M, shape[0], seed=52), synth.synth_x(M, shape[1], seed=53)
    got = to_np(ops.sdd(to_dev(a, dev), to_dev(b, dev), W))
    ref = O.sdd_at_b(O.bf16_round(a), O.bf16_round(b), m["row_idx"], m["col_idx"])
    assert_close_bf16(got, ref, f"dW {shape} M={M}")


_GROUP_SIZE_CASE = {}


def _group_size_case(M):
    """One ragged topology over three K segments with its operands and the oracle's gradient, computed once."""
    if M not in _GROUP_SIZE_CASE:
        m = synth.synth_matrix(16 * 200, 16 * 100, 0.3, seed=61, zipf_s=1.2)
        a, b = synth.synth_x(M, 16 * 200, seed=62 + M), synth.synth_x(M, 16 * 100, seed=63 + M)
        _GROUP_SIZE_CASE[M] = (m, a, b, O.sdd_at_b(O.bf16_round(a), O.bf16_round(b), m["row_idx"], m["col_idx"]))
    return _GROUP_SIZE_CASE[M]


@pytest.mark.parametrize("blocks_per_wave", [8, 10, 12, 14, 16, 18, 20, 22])
def test_sdd_every_group_size(dev, blocks_per_wave):
    """Each built group size (blocks per wavefront) against the oracle, on ragged rows over several K segments and
    several token ranges, and on a token count that ends inside a step."""
    for M in (600, 37):
        m, a, b, ref = _group_size_case(M)
        got = to_np(ops.sdd(to_dev(a, dev), to_dev(b, dev), synth.to_pack(m, dev), blocks_per_wave=blocks_per_wave))
        assert_close_bf16(got, ref, f"dW group size {blocks_per_wave} M={M}")
    with pytest.raises(ValueError):
        ops.sdd(to_dev(a, dev), to_dev(b, dev), synth.to_pack(m, dev), blocks_per_wave=9)


def test_sdd_exact_positions(dev):
    """One-hot operands: a single token with a single 1 in a and in b gives a single 1 in exactly one block element."""
    m = synth.synth_matrix(16 * 3, 16 * 5, 1.0, seed=1)
    W = synth.to_pack(m, dev)
    for tok, fa, fb in ((0, 0, 0), (5, 17, 33), (31, 47, 79), (40, 16, 15)):
        a = torch.zeros(41, 48, dtype=torch.bfloat16, device=dev); a[tok, fa] = 1.0
        b = torch.zeros(41, 80, dtype=torch.bfloat16, device=dev); b[tok, fb] = 1.0
        got = ops.sdd(a, b, W).float().cpu().numpy()
        want = np.zeros_like(got)
        j = int(np.nonzero((m["row_idx"] == fa // 16) & (m["col_idx"] == fb // 16))[0][0])
        want[j, fa % 16, fb % 16] = 1.0
        assert np.array_equal(got, want), (tok, fa, fb)


def test_sdd_edge_cases(dev):
    m = synth.synth_matrix(16 * 4, 16 * 6, 0.5, seed=2)
    W = synth.to_pack(m, dev)
    z = ops.sdd(torch.zeros(0, 64, dtype=torch.bfloat16, device=dev), torch.zeros(0, 96, dtype=torch.bfloat16, device=dev), W)
    assert z.shape == (W.nnz, 16, 16) and float(z.float().abs().max()) == 0.0
    with pytest.raises(ValueError):
        ops.sdd(torch.zeros(4, 64, dtype=torch.bfloat16, device=dev), torch.zeros(5, 96, dtype=torch.bfloat16, device=dev), W)
    with pytest.raises(ValueError):
        ops.sdd(torch.zeros(4, 96, dtype=torch.bfloat16, device=dev), torch.zeros(4, 96, dtype=torch.bfloat16, device=dev), W)
    # strided views of wider buffers
    a = torch.randn(50, 128, device=dev).to(torch.bfloat16)
    b = torch.randn(50, 192, device=dev).to(torch.bfloat16)
    got = to_np(ops.sdd(a[:, 64:], b[:, :96], W))
    ref = O.sdd_at_b(to_np(a[:, 64:]), to_np(b[:, :96]), m["row_idx"], m["col_idx"])
    assert_close_bf16(got, ref, "strided")


# ---------------------------------------------------------------------------------------------- training step

def _qat_layer(out_f, in_f, density, seed, dev, dtype=torch.float32):
    from mortar_amd.block_sparse import CMSBlockLinear
    g = torch.Generator().manual_seed(seed)
    lin = CMSBlockLinear(in_f, out_f, bias=False, dtype=dtype)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(out_f, in_f, generator=g) * 0.05)
    mask = torch.rand(out_f // 16, in_f // 16, generator=g) < density
    mask[torch.arange(out_f // 16), torch.randint(0, in_f // 16, (out_f // 16,), generator=g)] = True
    mask[torch.randint(0, out_f // 16, (in_f // 16,), generator=g), torch.arange(in_f // 16)] = True   # no empty column
    lin.set_block_mask(mask, 16)
    lin.carve(16)
    lin.enable_values_ternary(0.5)
    return lin.to(dev)


def _effective_dense(lin):
    """scale * q scattered to [out, in] in float64, with the scale rounded to bf16 as the kernels (and the reference's
    bf16 autocast) apply it."""
    d = lin.mortar_data.detach().float().cpu().numpy()
    q, s = O.ternary_quantize(d, lin._values_threshold)
    blocks = q.astype(np.float32) * O.bf16_round(np.float32(s))
    return O.to_dense(blocks, lin.mortar_row_indices.cpu().numpy(), lin.mortar_column_indices.cpu().numpy(),
                      (lin.out_features, lin.in_features)).astype(np.float64)


@pytest.mark.parametrize("M", [8, 300])
def test_qat_layer_forward_backward(dev, M):
    """A carved layer in values-ternary QAT: forward through the device-side re-pack, dX through the W^T pack, the
    gradient of mortar_data through the topology-restricted product (straight-through), then a second step after the
    values changed in place (the packs must follow)."""
    lin = _qat_layer(16 * 10, 16 * 7, 0.4, 61, dev)
    for step in range(2):
        W = _effective_dense(lin)
        x = synth.synth_x(M, lin.in_features, seed=62 + step)
        dy = synth.synth_x(M, lin.out_features, seed=64 + step)
        xt = to_dev(x, dev).requires_grad_(True)
        y = lin(xt)
        y.backward(to_dev(dy, dev))
        xb, dyb = O.bf16_round(x).astype(np.float64), O.bf16_round(dy).astype(np.float64)
        assert_close_bf16(to_np(y), (xb @ W.T).astype(np.float32), f"y step {step}")
        assert_close_bf16(to_np(xt.grad), (dyb @ W).astype(np.float32), f"dx step {step}")
        ref_dw = O.sdd_at_b(O.bf16_round(dy), O.bf16_round(x), lin.mortar_row_indices.cpu().numpy(),
                            lin.mortar_column_indices.cpu().numpy())
        assert lin.mortar_data.grad.shape == lin.mortar_data.shape and lin.mortar_data.grad.dtype == lin.mortar_data.dtype
        assert_close_bf16(to_np(lin.mortar_data.grad), ref_dw, f"d mortar_data step {step}")
        with torch.no_grad():                      # an optimiser step: same storage, new version
            lin.mortar_data.add_(lin.mortar_data.grad, alpha=-0.05)
            lin.mortar_data.grad = None


def test_qat_pack_follows_writes_through_data(dev):
    """Writes through ``mortar_data.data`` do not advance the parameter's version counter; the training forward re-encodes
    the values on every call, so forward, dX and dW all see the new values."""
    lin = _qat_layer(16 * 6, 16 * 5, 0.5, 66, dev)
    x = synth.synth_x(40, lin.in_features, seed=67)
    xt = to_dev(x, dev).requires_grad_(True)
    y0 = lin(xt)
    v0 = lin.mortar_data._version
    lin.mortar_data.data.mul_(-1.0)
    assert lin.mortar_data._version == v0                            # the write is invisible to the version key
    y1 = lin(xt)
    assert torch.equal(y1, -y0)
    dy = to_dev(synth.synth_x(40, lin.out_features, seed=68), dev)
    y1.backward(dy)
    W = _effective_dense(lin)
    assert_close_bf16(to_np(xt.grad), (O.bf16_round(to_np(dy)).astype(np.float64) @ W).astype(np.float32), "dx after .data write")
    lin.mortar_data.data.mul_(-1.0)
    with torch.no_grad():                                            # the inference path follows explicit invalidation
        lin.invalidate_pack()
        assert torch.equal(lin(xt.detach()), y0)


def test_stk_dds_fp32_effective_data_and_the_ternary_form(dev):
    """The reference's own caller in fp32: _mortar_effective_data() = d + (scale*q - d).detach() is +-s only to within an
    fp32 ulp (several distinct magnitudes).  stk_dds multiplies it as it is (cast to bf16); stk_dds_ternary runs it on the
    ternary kernels and must accept it; data that is NOT ternary makes stk_dds_ternary's result NaN in the same call and
    raises -- synchronously in the first call on a topology, through the device flag later (stk_check waits for it) --
    while stk_dds just multiplies it."""
    import mortar_amd
    from mortar_amd import stk
    from mortar_amd.stk import stk_dds_ternary
    lin = _qat_layer(16 * 8, 16 * 6, 0.5, 86, dev)
    eff = lin._mortar_effective_data().detach()
    assert eff.dtype == torch.float32
    mags = torch.unique(eff.abs()[eff != 0])
    assert mags.numel() > 1 and float(mags.max() / mags.min()) < 1 + 1e-5      # really not bit-equal magnitudes
    z32, z16 = torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int16, device=dev)
    args = (lin.mortar_offsets, lin.mortar_row_indices, lin.mortar_column_indices, z32, z16, z32)
    x = synth.synth_x(30, lin.in_features, seed=87)
    want = (O.bf16_round(x).astype(np.float64) @ _effective_dense(lin).T).astype(np.float32)
    for op in (mortar_amd.stk_dds, stk_dds_ternary):
        y = op(to_dev(x, dev), eff, *args, lin.in_features, lin.out_features, True)
        assert_close_bf16(to_np(y), want, "fp32 effective data")
        yb = op(to_dev(x, dev), eff.to(torch.bfloat16), *args, lin.in_features, lin.out_features, True)
        assert torch.equal(y, yb)
    ones = torch.ones(5, lin.out_features, dtype=torch.bfloat16, device=dev)
    dx0 = stk_dds_ternary(ones, eff, *args, lin.out_features, lin.in_features, False)             # first call on the W^T pack (waits)
    assert_close_bf16(to_np(dx0), to_np(mortar_amd.stk_dds(ones, eff, *args, lin.out_features, lin.in_features, False)), "dX both forms", ulps=4)
    stk.stk_check()                                                   # nothing to report so far
    # same topology, later call, data that is NOT ternary: no wait in the call itself, the flag is raised on the device
    bad = eff.clone(); bad[3, 2, 1] = 0.37 * float(mags[0])
    ybad = stk_dds_ternary(to_dev(x, dev), bad, *args, lin.in_features, lin.out_features, True)
    assert bool(torch.isnan(ybad).all())                              # ...and the product of that call is unusable: all NaN
    with pytest.raises(ValueError, match="not ternary"):
        stk.stk_check()
    stk.stk_check()                                                   # reported once, then clean again
    ybad = stk_dds_ternary(to_dev(x.astype(np.float32), dev).float(), bad, *args, lin.in_features, lin.out_features, True)
    assert ybad.dtype == torch.float32 and bool(torch.isnan(ybad).all())
    dxbad = stk_dds_ternary(ones, bad, *args, lin.out_features, lin.in_features, False)           # the dX product through the W^T pack
    assert bool(torch.isnan(dxbad).all())
    torch.cuda.synchronize()
    with pytest.raises(ValueError, match="earlier call"):             # the next call finds the flag on the host
        stk_dds_ternary(to_dev(x, dev), eff, *args, lin.in_features, lin.out_features, True)
    y2 = stk_dds_ternary(to_dev(x, dev), eff, *args, lin.in_features, lin.out_features, True)
    assert_close_bf16(to_np(y2), want, "after the report")
    with pytest.raises(ValueError, match="not ternary"):              # the W^T pack keeps its own words
        stk.stk_check()
    dx = stk_dds_ternary(ones, eff, *args, lin.out_features, lin.in_features, False)
    assert torch.equal(dx, dx0)
    # the general operator multiplies the non-ternary data as the reference does
    yg = mortar_amd.stk_dds(to_dev(x, dev), bad, *args, lin.in_features, lin.out_features, True)
    bad_dense = O.to_dense(O.bf16_round(bad.cpu().numpy()), lin.mortar_row_indices.cpu().numpy(), lin.mortar_column_indices.cpu().numpy(),
                           (lin.out_features, lin.in_features)).astype(np.float64)
    assert_close_bf16(to_np(yg), (O.bf16_round(x).astype(np.float64) @ bad_dense.T).astype(np.float32), "non-ternary data, general operator")
    # a fresh topology sees the error in its first call
    m = synth.synth_matrix(64, 64, 0.5, seed=88)
    t = lambda a: torch.from_numpy(a).to(dev)
    with pytest.raises(ValueError, match="not ternary"):
        stk_dds_ternary(torch.zeros(4, 64, dtype=torch.bfloat16, device=dev), torch.randn(m["col_idx"].size, 16, 16, device=dev),
                        t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32, 64, 64, True)


def test_qat_mlp_trains_layer_by_layer(dev):
    """The SwiGLU MLP with QAT layers and autograd on: same value as the fused inference path, gradients reach the
    input and both block-value tensors."""
    from mortar_amd.mlp import _SwiGLUMortar
    d_model, d_ff = 16 * 6, 16 * 10
    mlp = _SwiGLUMortar(d_model, d_ff)
    mlp.gate_up._cms = _qat_layer(2 * d_ff, d_model, 0.5, 71, dev)
    mlp.down._cms = _qat_layer(d_model, d_ff, 0.5, 72, dev)
    mlp = mlp.to(dev)
    x = to_dev(synth.synth_x(50, d_model, seed=73), dev)
    with torch.no_grad():
        y_inf = mlp(x)
    xg = x.clone().requires_grad_(True)
    y = mlp(xg)
    assert_close_bf16(to_np(y), to_np(y_inf), "train path vs fused path", ulps=8)
    y.float().pow(2).sum().backward()
    for name, g in (("x", xg.grad), ("gate_up", mlp.gate_up._cms.mortar_data.grad), ("down", mlp.down._cms.mortar_data.grad)):
        assert g is not None and torch.isfinite(g.float()).all() and float(g.float().abs().max()) > 0, name
    # against a dense torch twin with the same effective weights (fp32 autograd)
    Wg = torch.from_numpy(_effective_dense(mlp.gate_up._cms)).float().to(dev)
    Wd = torch.from_numpy(_effective_dense(mlp.down._cms)).float().to(dev)
    xr = x.float().clone().requires_grad_(True)
    gu = xr @ Wg.T
    h = torch.nn.functional.silu(gu[:, :d_ff]) * gu[:, d_ff:]
    yr = h @ Wd.T
    yr.pow(2).sum().backward()
    # five bf16 roundings lie between the two chains: compare in the large (max error 3e-2 of the largest entry, cosine)
    got, ref = to_np(xg.grad).astype(np.float64), to_np(xr.grad).astype(np.float64)
    assert np.abs(got - ref).max() <= 3e-2 * np.abs(ref).max()
    assert (got * ref).sum() / np.sqrt((got * got).sum() * (ref * ref).sum()) > 0.9995


def test_stk_dds_operator_autograd(dev):
    """The custom op's registered backward: dlhs through the other orientation, ddata through stk_sdd_at_b."""
    import mortar_amd
    m = synth.synth_matrix(16 * 8, 16 * 6, 0.5, seed=81)
    t = lambda a: torch.from_numpy(a).to(dev)
    data = t(O.effective_blocks(m["codes"], m["scales"])).to(torch.bfloat16).requires_grad_(True)
    dense = O.to_dense(data.detach().float().cpu().numpy(), m["row_idx"], m["col_idx"], (128, 96)).astype(np.float64)
    z32, z16 = torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int16, device=dev)
    args = (t(m["offsets"]), t(m["row_idx"]), t(m["col_idx"]), z32, z16, z32)
    x, dy = synth.synth_x(70, 96, seed=82), synth.synth_x(70, 128, seed=83)
    xt = to_dev(x, dev).requires_grad_(True)
    y = mortar_amd.stk_dds(xt, data, *args, 96, 128, True)
    y.backward(to_dev(dy, dev))
    assert_close_bf16(to_np(xt.grad), (O.bf16_round(dy) @ dense).astype(np.float32), "dlhs")
    assert data.grad.shape == data.shape and data.grad.dtype == torch.bfloat16
    assert_close_bf16(to_np(data.grad), O.sdd_at_b(O.bf16_round(dy), O.bf16_round(x), m["row_idx"], m["col_idx"]), "ddata")
    direct = mortar_amd.stk_sdd_at_b(to_dev(dy, dev), to_dev(x, dev), data.detach(), *args[:3])
    assert torch.equal(direct, data.grad)


@pytest.mark.parametrize("M,d_ff", [(1, 16), (70, 16 * 10), (300, 16 * 352)])
def test_swiglu_training_kernels(dev, M, d_ff):
    """The stand-alone SwiGLU and its derivative against the oracle (bf16 tensors rounded where the eager graph has them)."""
    gu = synth.synth_x(M, 2 * d_ff, seed=91) * 2.0
    dh = synth.synth_x(M, d_ff, seed=92)
    gt, dt = to_dev(gu, dev), to_dev(dh, dev)
    gb, db = O.bf16_round(gu), O.bf16_round(dh)
    assert_close_bf16(to_np(ops.swiglu(gt)), O.swiglu(gb), "swiglu", ulps=2)
    assert_close_bf16(to_np(ops.swiglu_backward(gt, dt)), O.swiglu_backward(gb, db), "swiglu backward", ulps=3)
    # the fused gate_up epilogue and the stand-alone kernel round alike: same bits from the same gate_up output
    wide = torch.zeros(M, 2 * d_ff + 32, dtype=torch.bfloat16, device=dev)
    wide[:, 8:8 + 2 * d_ff] = gt
    assert torch.equal(ops.swiglu(wide[:, 8:8 + 2 * d_ff]), ops.swiglu(gt))
    with pytest.raises(ValueError):
        ops.swiglu_backward(gt, dt[:, :-8])


def test_qat_mlp_single_op_training_step(dev):
    """The whole MLP as one autograd op (no router): value equals the fused inference path bit for bit where the
    rounding points agree, and all three gradients match the layer-by-layer path."""
    from mortar_amd.mlp import _SwiGLUMortar
    d_model, d_ff = 16 * 6, 16 * 10
    mlp = _SwiGLUMortar(d_model, d_ff)
    mlp.gate_up._cms = _qat_layer(2 * d_ff, d_model, 0.5, 71, dev)
    mlp.down._cms = _qat_layer(d_model, d_ff, 0.5, 72, dev)
    mlp = mlp.to(dev)
    x = to_dev(synth.synth_x(90, d_model, seed=73), dev)
    dy = to_dev(synth.synth_x(90, d_model, seed=74), dev)
    with torch.no_grad():
        y_inf = mlp(x)
    xg = x.clone().requires_grad_(True)
    y = mlp(xg)
    fns, node = [], y.grad_fn
    while node is not None and len(fns) < 4:
        fns.append(type(node).__name__)
        node = node.next_functions[0][0] if node.next_functions else None
    assert any("SwiGLUMortarFn" in f for f in fns), fns
    assert_close_bf16(to_np(y), to_np(y_inf), "single-op forward vs fused inference", ulps=4)
    y.backward(dy)
    got = [xg.grad.clone(), mlp.gate_up._cms.mortar_data.grad.clone(), mlp.down._cms.mortar_data.grad.clone()]
    for p in (mlp.gate_up._cms.mortar_data, mlp.down._cms.mortar_data):
        p.grad = None
    # layer by layer (carved linear -> torch SwiGLU -> carved linear), forced by a dummy gate of ones
    xr = x.clone().requires_grad_(True)
    gu = mlp.gate_up(xr)
    h = torch.nn.functional.silu(gu[:, :d_ff]) * gu[:, d_ff:]
    mlp.down(h).backward(dy)
    ref = [xr.grad, mlp.gate_up._cms.mortar_data.grad, mlp.down._cms.mortar_data.grad]
    for name, a, b in zip(("dx", "d gate_up", "d down"), got, ref):
        assert_close_bf16(to_np(a), to_np(b), name, ulps=6)


def test_full_size_backward_adjoint_identities(dev):
    """Headline shapes (d_model 2048, d_ff 5632, 25 %, 4096 tokens): the oracle cannot run these in seconds, so the
    backward is checked through the adjoint identities of y = x W^T, which hold for any size:
    <dY, x W^T> = <dY W, x> = <dW, W>, with every product taken from the HIP path and the sums in float64."""
    spec = synth.synth_mlp(2048, 5632, 0.25, seed=0)
    M = 4096
    for name in ("gate_up", "down"):
        m = spec[name]
        out_f, in_f = m["shape"]
        nnz = m["col_idx"].size
        W = MortarPack(None, None, m["col_idx"], m["offsets"], out_f, in_f, dev)
        vals = (torch.randn(nnz, 16, 16, device=dev, generator=torch.Generator(device=dev).manual_seed(5)) * 0.05).to(torch.bfloat16)
        s = W.requantize(vals, per_block=True)
        Wt = W.transposed()
        Wt.requantize(vals, per_block=True, transpose=True)
        x = to_dev(synth.synth_x(M, in_f, seed=6), dev)
        dy = to_dev(synth.synth_x(M, out_f, seed=7), dev)
        y, dx, dw = ops.spmm(x, W), ops.spmm(dy, Wt), ops.sdd(dy, x, W)
        codes = torch.from_numpy(decode_blocks(W.codes.cpu().numpy().view(np.uint32))).to(dev)
        w_eff = codes.double() * s.to(torch.bfloat16).double()[:, None, None]
        a = float((dy.double() * y.double()).sum())
        b = float((dx.double() * x.double()).sum())
        c = float((dw.double() * w_eff).sum())
        scale = float(dy.double().pow(2).sum().sqrt() * y.double().pow(2).sum().sqrt())      # Cauchy-Schwarz size of the sum
        assert abs(a - b) <= 2e-3 * scale and abs(a - c) <= 2e-3 * scale, (name, a, b, c, scale)
        # and dW of the full-size launch equals dW of two half-batches added (linearity in the token dimension)
        half = ops.sdd(dy[:2048], x[:2048], W).float() + ops.sdd(dy[2048:], x[2048:], W).float()
        assert float((dw.float() - half).abs().max()) <= 2.0 ** -6 * float(dw.float().abs().max())


def test_training_golden_fixture(dev):
    """The HIP training path against the committed vectors (tests/golden/train_slice.npz): device-side ternarisation,
    forward, dX through the W^T pack, dW on the topology, SwiGLU and its derivative."""
    import golden_util as G
    z = G.load("train_slice.npz")
    shape = tuple(int(v) for v in z["shape"])
    bits = lambda name: torch.from_numpy(z[name].view(np.int16)).view(torch.bfloat16).to(dev)
    vals, x, dy = bits("values_bits"), bits("x_bits"), bits("dy_bits")
    W = MortarPack(None, None, z["col_idx"], z["offsets"], shape[0], shape[1], dev)
    s = W.requantize(vals)
    np.testing.assert_allclose(s.cpu().numpy(), z["scale_bits"].view(np.float32), rtol=4e-7, atol=0)
    got = decode_blocks(W.codes.cpu().numpy().view(np.uint32))
    v = O.bf16_from_bits(z["values_bits"])
    off = np.abs(np.abs(v / z["scale_bits"].view(np.float32)[0]) - 0.5) > 1e-5          # away from the threshold itself
    assert np.array_equal(got[off], z["codes"][off]) and (got != z["codes"]).mean() < 1e-5
    Wb = MortarPack(None, None, z["col_idx"], z["offsets"], shape[0], shape[1], dev)
    sb = Wb.requantize(vals, per_block=True)
    np.testing.assert_allclose(sb.cpu().numpy(), z["scale_per_block_bits"].view(np.float32), rtol=4e-7, atol=0)
    gotb = decode_blocks(Wb.codes.cpu().numpy().view(np.uint32))
    assert (gotb != z["codes_per_block"]).mean() < 1e-5
    Wt = W.transposed()
    Wt.requantize(vals, scale=s, transpose=True)
    assert_close_bf16(to_np(ops.spmm(x, W)), O.bf16_from_bits(z["y_bits"]), "y")
    assert_close_bf16(to_np(ops.spmm(dy, Wt)), O.bf16_from_bits(z["dx_bits"]), "dx")
    assert_close_bf16(to_np(ops.sdd(dy, x, W)), O.bf16_from_bits(z["dw_bits"]), "dW")
    assert_close_bf16(to_np(ops.swiglu(bits("gu_bits"))), O.bf16_from_bits(z["h_bits"]), "h")
    assert_close_bf16(to_np(ops.swiglu_backward(bits("gu_bits"), bits("dh_bits"))), O.bf16_from_bits(z["dgu_bits"]), "dgu", ulps=3)


@pytest.mark.parametrize("packed", [True, False])
def test_layer_carved_at_blocking_128_runs_through_the_recut_pack(dev, packed):
    """The reference's default carve (blocking 128, block_sparse.py:810; pruning.py:85,248): a layer pruned on 16-tiles,
    carved at 128 and either packed (deploy_quant.py:344-374) or left in values-ternary mode is re-cut into 16 x 16 blocks
    at pack time; prefill and decode forwards against the dense float64 product of its effective weight."""
    import mortar_amd
    torch.manual_seed(21)
    lin = mortar_amd.MortarLinear(512, 384, bias=False)
    rng = np.random.default_rng(22)
    tiles = rng.random((24, 32)) < 0.3
    tiles[::8, 0] = True                                                   # every 128-row keeps a block
    lin._cms._prune_mask = torch.from_numpy(tiles)
    lin.carve(128)
    cms = lin._cms
    if packed:
        mortar_amd.pack_mortar_ternary(cms, 0.5)
    else:
        cms.enable_values_ternary(0.5)
    lin.to(dev)
    eff = cms._mortar_effective_data().detach().float().cpu().numpy()
    if not packed:                                                         # the kernels multiply bf16(scale) * code
        sc = float(cms.mortar_data.detach().float().abs().mean().clamp(min=1e-8))
        eff = np.sign(eff) * O.bf16_round(np.array([sc], np.float32))[0]
    dense = O.to_dense(eff, cms.mortar_row_indices.cpu().numpy(), cms.mortar_column_indices.cpu().numpy(), (384, 512), 128)
    W = cms.mortar_pack()
    assert W.nnz < int(cms.mortar_row_indices.numel()) * 64                # pruned tiles inside kept blocks were dropped
    for M in (200, 3):
        x = synth.synth_x(M, 512, seed=23 + M)
        with torch.no_grad():
            y = lin(to_dev(x, dev))
        assert_close_bf16(to_np(y), (O.bf16_round(x).astype(np.float64) @ dense.astype(np.float64).T).astype(np.float32), f"blocking 128, M={M}")
    if not packed:
        with pytest.raises(RuntimeError, match="blocking 128"):
            lin(to_dev(x, dev).requires_grad_(True))
