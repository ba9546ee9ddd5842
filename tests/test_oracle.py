"""Pins the CPU oracle WITHOUT the reference: closed forms, brute force, library routines, invariants.
Each check is chosen so that a plausible mistake (dropped term, wrong index, transposed operand) fails."""
import itertools

import numpy as np
import pytest

from oracle import c_oracle
from oracle import mortar_oracle as O


def rand_case(Rb, Cb, density, seed, blk=16):
    rng = np.random.default_rng(seed)
    mask = rng.random((Rb, Cb)) < density
    mask[np.arange(Rb), rng.integers(0, Cb, Rb)] = True
    w = rng.standard_normal((Rb * blk, Cb * blk)).astype(np.float32)
    return w, mask


# ---- carve -------------------------------------------------------------------------------------------

def test_carve_layout_closed_form():
    w, mask = rand_case(5, 7, 0.4, 0)
    c = O.carve(w, mask, 16)
    # row-major nonzero order, int16/int32 dtypes, offsets = exclusive cumsum (block_sparse.py:874-883)
    rows, cols = np.nonzero(mask)
    assert c["mortar_row_indices"].dtype == np.int16 and c["mortar_column_indices"].dtype == np.int16
    assert c["mortar_offsets"].dtype == np.int32
    assert np.array_equal(c["mortar_row_indices"], rows) and np.array_equal(c["mortar_column_indices"], cols)
    assert np.array_equal(c["mortar_offsets"], np.concatenate([[0], np.cumsum(mask.sum(1))]))
    # element order inside a block: data[j, lr, c] = W[row*blk+lr, col*blk+c] -- checked element by element
    for j in (0, len(rows) // 2, len(rows) - 1):
        for lr, cc in ((0, 0), (3, 11), (15, 15), (7, 2)):
            assert c["mortar_data"][j, lr, cc] == w[rows[j] * 16 + lr, cols[j] * 16 + cc]


def test_carve_scatter_round_trip():
    w, mask = rand_case(6, 9, 0.3, 1)
    c = O.carve(w, mask, 16)
    dense = O.to_dense(c["mortar_data"], c["mortar_row_indices"], c["mortar_column_indices"], w.shape, 16)
    expect = w * np.kron(mask, np.ones((16, 16), dtype=np.float32))
    assert np.array_equal(dense, expect)


def test_carve_errors():
    w, mask = rand_case(4, 4, 0.5, 2)
    mask[2, :] = False
    with pytest.raises(RuntimeError):
        O.carve(w, mask, 16)
    with pytest.raises(ValueError):
        O.carve(w[:-1], mask, 16)


def test_transpose_meta_invariants():
    w, mask = rand_case(6, 5, 0.5, 3)
    c = O.carve(w, mask, 16)
    ct, ot, bt = c["mortar_column_indices_t"], c["mortar_offsets_t"], c["mortar_block_offsets_t"]
    assert np.array_equal(ot, np.concatenate([[0], np.cumsum(mask.sum(0))]))
    assert sorted(bt.tolist()) == list(range(mask.sum()))                      # a permutation of the blocks
    for col in range(5):
        js = bt[ot[col]:ot[col + 1]]
        assert (c["mortar_column_indices"][js] == col).all()
        assert np.array_equal(ct[ot[col]:ot[col + 1]], c["mortar_row_indices"][js])


# ---- ternary / pack ----------------------------------------------------------------------------------

def test_ternary_quantize_rule():
    # known answers written out by hand (deploy_quant.py:91-94): sum|w| = 8 over 8 entries, so the scale is exactly
    # 1.0 and the entries +-0.5 sit exactly ON the threshold 0.5 * mean|w|: the compare is strict, their code is 0
    w = np.array([0.5, -0.5, 1.5, -1.5, 1.0, -1.0, 2.0, 0.0], dtype=np.float32)
    q, s = O.ternary_quantize(w)
    assert s == np.float32(1.0)
    assert q.tolist() == [0, 0, 1, -1, 1, -1, 1, 0]
    # the same values times 4 (power of two: every quotient is exact): scale 4, entries +-2 on the threshold
    q4, s4 = O.ternary_quantize(w * np.float32(4.0))
    assert s4 == np.float32(4.0) and q4.tolist() == [0, 0, 1, -1, 1, -1, 1, 0]
    # one ulp above the threshold is kept, one ulp below is dropped
    w2 = w.copy(); w2[0] = np.nextafter(np.float32(0.5), np.float32(1)); w2[1] = -np.nextafter(np.float32(0.5), np.float32(0))
    w2[7] = np.float32(8.0) - np.abs(w2[:7]).sum(dtype=np.float32)            # keeps sum|w| = 8 to within an ulp
    q2, s2 = O.ternary_quantize(w2)
    assert abs(float(s2) - 1.0) < 1e-6 and q2[:2].tolist() == [1, 0]
    # a threshold other than the default moves the cut with it
    assert O.ternary_quantize(w, threshold=1.0)[0].tolist() == [0, 0, 1, -1, 0, 0, 1, 0]
    # the per-block form applies the same strict rule with each block's own mean
    wb = np.zeros((2, 16, 16), np.float32)
    wb[0] = 2.0; wb[0, 0, :8] = 1.0; wb[0, 1, :8] = -3.0     # mean|w| = (240*2 + 8 + 24) / 256 = 2.0: the 1.0s sit on the cut
    wb[1] = -0.25; wb[1, 5, 5] = 0.125                       # mean = (255*0.25 + 0.125) / 256: 0.125 is just above half of it
    qb, sb = O.ternary_quantize_per_block(wb)
    assert sb[0] == np.float32(2.0) and (qb[0, 0, :8] == 0).all() and (qb[0, 1, :8] == -1).all() and (qb[0, 2:] == 1).all()
    assert qb[1, 5, 5] == 1 and (qb[1].sum() == -255 + 1)
    # invariant of tests/test_lifecycle_tst_qat.py:100-105: every non-zero effective weight has one magnitude
    eff = q.astype(np.float32) * s
    assert len(np.unique(np.abs(eff[eff != 0]))) == 1
    assert O.ternary_quantize(np.zeros(8, np.float32))[1] == np.float32(1e-8)  # clamp (deploy_quant.py:91)
    assert O.ternary_quantize_per_block(np.zeros((1, 16, 16), np.float32))[1][0] == np.float32(1e-6)  # block_sparse.py:397


def test_ternary_per_block_is_per_tensor_on_each_block():
    rng = np.random.default_rng(4)
    w = rng.standard_normal((5, 16, 16)).astype(np.float32)
    q, s = O.ternary_quantize_per_block(w)
    for j in range(5):
        qj, sj = O.ternary_quantize(w[j])
        assert np.array_equal(q[j], qj) and np.isclose(s[j], sj, rtol=1e-6)


def test_pack_exhaustive_bytes():
    # all 256 byte values: decode by definition (2 bits each, little-endian, minus one)
    for b in range(256):
        codes = O.unpack_ternary(np.array([b], dtype=np.uint8), 4)
        assert codes.tolist() == [((b >> (2 * i)) & 3) - 1 for i in range(4)]
    # all 81 valid quadruples round-trip, and the byte is u0 + 4*u1 + 16*u2 + 64*u3
    for quad in itertools.product((-1, 0, 1), repeat=4):
        p = O.pack_ternary_codes(np.array(quad, dtype=np.int8))
        assert p.tolist() == [sum((c + 1) << (2 * i) for i, c in enumerate(quad))]
        assert O.unpack_ternary(p, 4).tolist() == list(quad)
    # padding to a multiple of four with stored value 0
    assert O.pack_ternary_codes(np.array([1, 1, 1, 1, 1], np.int8)).tolist() == [0xAA, 0x02]


def test_pack_strips_layout():
    rng = np.random.default_rng(5)
    codes = rng.integers(-1, 2, size=(3, 16, 16)).astype(np.int8)
    s = O.pack_strips(codes)
    assert s.shape == (3, 16, 4)
    for j, lr, b in ((0, 0, 0), (1, 5, 3), (2, 15, 2)):
        got = [((int(s[j, lr, b]) >> (2 * k)) & 3) - 1 for k in range(4)]
        assert got == [codes[j, lr, b + 4 * k] for k in range(4)]            # columns {b, 4+b, 8+b, 12+b}


def test_work_list_partitions_rows():
    offsets = np.array([0, 3, 3 + 9, 12 + 4, 16 + 1], dtype=np.int32)
    ent, nmax, cnts = O.work_list(offsets, cb=4)
    assert cnts.tolist() == [1, 3, 1, 1] and nmax == 3
    for r in range(4):
        e = ent[:, ent[0] == r]
        assert e[2].tolist() == list(range(cnts[r]))
        assert e[1].tolist() == [offsets[r] + 4 * s for s in range(cnts[r])]


# ---- SpMM ---------------------------------------------------------------------------------------------

def make_mat(Rb, Cb, density, seed):
    rng = np.random.default_rng(seed)
    mask = rng.random((Rb, Cb)) < density
    mask[np.arange(Rb), rng.integers(0, Cb, Rb)] = True
    rows, cols = np.nonzero(mask)
    nnz = len(rows)
    return dict(codes=rng.integers(-1, 2, (nnz, 16, 16)).astype(np.int8),
                scales=rng.uniform(0.01, 0.1, nnz).astype(np.float32),
                col_idx=cols.astype(np.int16), row_idx=rows.astype(np.int16),
                offsets=np.concatenate([[0], np.cumsum(mask.sum(1))]).astype(np.int32), shape=(Rb * 16, Cb * 16))


def xbf(M, K, seed):
    return O.bf16_round(np.random.default_rng(seed).standard_normal((M, K)).astype(np.float32))


def test_spmm_equals_dense_scatter_matmul():
    m = make_mat(7, 9, 0.35, 10)
    x = xbf(13, 9 * 16, 11)
    y = O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"], round_out=False)
    W = O.to_dense(m["codes"].astype(np.float64) * O.bf16_round(m["scales"]).astype(np.float64)[:, None, None],
                   m["row_idx"], m["col_idx"], m["shape"])
    ref = x.astype(np.float64) @ W.T                                          # library routine, W not transposed twice
    assert np.allclose(y, ref, rtol=1e-6, atol=1e-6)
    # a transposed block (data[j,c,n] instead of data[j,n,c]) must NOT pass
    bad = O.bcsr_spmm(x, m["codes"].transpose(0, 2, 1), m["scales"], m["col_idx"], m["offsets"], round_out=False)
    assert not np.allclose(bad, ref, rtol=1e-3, atol=1e-3)


def test_spmm_special_cases():
    rng = np.random.default_rng(12)
    # density 1, scale 1 == dense GEMM with the ternary matrix
    Rb, Cb = 3, 4
    codes = rng.integers(-1, 2, (Rb * Cb, 16, 16)).astype(np.int8)
    col = np.tile(np.arange(Cb), Rb).astype(np.int16)
    row = np.repeat(np.arange(Rb), Cb).astype(np.int16)
    off = (np.arange(Rb + 1) * Cb).astype(np.int32)
    x = xbf(5, Cb * 16, 13)
    W = O.to_dense(codes.astype(np.float32), row, col, (Rb * 16, Cb * 16))
    y = O.bcsr_spmm(x, codes, np.float32(1.0), col, off, round_out=False)
    assert np.allclose(y, x @ W.T, atol=1e-5)
    # identity blocks on a block permutation: output block r == scale_r * input block perm[r]
    perm = np.array([2, 0, 3, 1])
    eye = np.tile(np.eye(16, dtype=np.int8), (4, 1, 1))
    s = np.array([0.5, 0.25, 2.0, 1.0], np.float32)
    y = O.bcsr_spmm(x, eye, s, perm.astype(np.int16), np.arange(5, dtype=np.int32), round_out=False)
    for r in range(4):
        assert np.allclose(y[:, r * 16:(r + 1) * 16], s[r] * x[:, perm[r] * 16:(perm[r] + 1) * 16])
    # all-zero codes -> zeros ; scale rounded to bf16 (0.1 is not bf16-representable)
    assert not O.bcsr_spmm(x, np.zeros_like(eye), s, perm.astype(np.int16), np.arange(5, dtype=np.int32)).any()
    y01 = O.bcsr_spmm(x, eye[:1], np.float32(0.1), np.array([0], np.int16), np.array([0, 1], np.int32), round_out=False)
    assert np.allclose(y01, O.bf16_round(np.float32(0.1)) * x[:, :16], rtol=1e-7)
    assert not np.allclose(y01, np.float32(0.1) * x[:, :16], rtol=1e-5)


def test_c_oracle_matches_numpy_oracle():
    m = make_mat(8, 12, 0.3, 20)
    x = xbf(9, 12 * 16, 21)
    ynp = O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"])
    yc = O.bf16_from_bits(c_oracle.bcsr_spmm_bf16(O.bf16_bits(x), m["codes"], m["scales"], m["col_idx"], m["offsets"]))
    # fp32 vs float64 accumulation may flip a bf16 rounding: allow 1 ulp on < 1 % of entries
    diff = np.abs(ynp - yc)
    assert (diff <= np.abs(ynp) * 2 ** -7 + 1e-6).all()
    assert (diff > 0).mean() < 0.01


def test_swiglu_mlp_against_dense():
    gu, dn = make_mat(2 * 6, 4, 0.5, 30), make_mat(4, 6, 0.5, 31)
    x = xbf(11, 64, 32)
    r = O.swiglu_mlp(x, gu, dn)
    Wg = O.to_dense(O.effective_blocks(gu["codes"], gu["scales"]), gu["row_idx"], gu["col_idx"], gu["shape"])
    g_u = O.bf16_round((x.astype(np.float64) @ Wg.astype(np.float64).T).astype(np.float32))
    g, u = g_u[:, :96], g_u[:, 96:]
    sig = 1.0 / (1.0 + np.exp(-g.astype(np.float64)))
    h = O.bf16_round(O.bf16_round((g * sig).astype(np.float32)) * u)
    assert np.array_equal(r["h"], h)
    Wd = O.to_dense(O.effective_blocks(dn["codes"], dn["scales"]), dn["row_idx"], dn["col_idx"], dn["shape"])
    y = O.bf16_round((h.astype(np.float64) @ Wd.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(r["y"], y)
    # gates: per-cluster multiply; gate 0 kills the cluster, gate 1 leaves it
    gates = np.zeros((11, 6), np.float32); gates[:, 1] = 1.0
    rg = O.swiglu_mlp(x, gu, dn, gates=gates)
    assert not rg["h"][:, :16].any() and np.array_equal(rg["h"][:, 16:32], h[:, 16:32]) and not rg["h"][:, 32:].any()
    gc, hc, yc = c_oracle.mlp_bf16(O.bf16_bits(x), gu, dn, 96, gates=gates)
    assert np.abs(O.bf16_from_bits(yc) - rg["y"]).max() <= np.abs(rg["y"]).max() * 2 ** -6


def test_decode_gemv_form_equals_spmm_unrounded():
    m = make_mat(5, 8, 0.4, 40)
    # with bf16-representable scales the decode form and the prefill form are the same sums
    m["scales"] = O.bf16_round(m["scales"])
    x = xbf(3, 128, 41)
    a = O.mortar_gemv(x, m["codes"], m["scales"], m["col_idx"], m["offsets"])
    b = O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"], round_out=False)
    assert np.allclose(a, b, rtol=1e-6, atol=1e-6)


def test_decode_gemv_keeps_the_fp32_scale_unrounded():
    """What separates the engine's GEMV from the prefill product (fused_decode_step.py:1335, 1441-1459): the scale is
    fp32, is NOT rounded to bf16, and multiplies the block's sum.  Hand-computed cases with scales that bf16 cannot
    hold (0.1 -> 0.10009765625 in bf16, 0.3 -> 0.30078125)."""
    eye = np.eye(16, dtype=np.int8)[None]
    x = np.arange(1, 17, dtype=np.float32)[None] / 4                      # 0.25 .. 4.0, exact in bf16
    s01 = np.float32(0.1)
    y = O.mortar_gemv(x, eye, np.array([s01]), np.array([0], np.int16), np.array([0, 1], np.int32))
    want = (x.astype(np.float64) * float(s01)).astype(np.float32)          # float32(0.1) * x, correctly rounded
    np.testing.assert_allclose(y, want, rtol=1e-7, atol=0)
    rounded = x * O.bf16_round(np.array([s01]))[0]                         # what a bf16 scale would give: 9.8e-4 off
    assert (np.abs(y - rounded) > 5e-4 * np.abs(y)).all()
    # the prefill product, by contrast, does round the scale (deploy_quant.py:367-369)
    yp = O.bcsr_spmm(x, eye, np.array([s01]), np.array([0], np.int16), np.array([0, 1], np.int32), round_out=False)
    np.testing.assert_allclose(yp, rounded, rtol=1e-7)
    # two blocks in one row, scales 0.1 and 0.3, codes +identity and -identity on block-columns 2 and 0:
    # y[n] = 0.1 * x[32 + n] - 0.3 * x[n]
    x2 = np.zeros((1, 48), np.float32); x2[0, 32:48] = 2.0; x2[0, 0:16] = np.arange(16) / 8
    codes = np.concatenate([-eye, eye])                                   # CSR order: ascending column (0 then 2)
    y2 = O.mortar_gemv(x2, codes, np.array([0.3, 0.1], np.float32), np.array([0, 2], np.int16), np.array([0, 2], np.int32))
    hand = float(np.float32(0.1)) * 2.0 - float(np.float32(0.3)) * (np.arange(16) / 8)
    np.testing.assert_allclose(y2[0], hand.astype(np.float32), rtol=2e-7, atol=1e-8)
    # scale multiplies the SUM of the block (codes with several non-zeros per row): row n = x[n] + x[n+1 mod 16]
    two = (np.eye(16, dtype=np.int8) + np.roll(np.eye(16, dtype=np.int8), 1, axis=1))[None]
    y3 = O.mortar_gemv(x, two, np.array([s01]), np.array([0], np.int16), np.array([0, 1], np.int32))
    hand3 = float(s01) * (x[0].astype(np.float64) + np.roll(x[0].astype(np.float64), -1))
    np.testing.assert_allclose(y3[0], hand3.astype(np.float32), rtol=2e-7)


def test_decode_gemv_flags_are_per_stream():
    """fused_decode_step.py:1378-1393: stream b reads ROWACT[b, r] and COLACT[b, cb] only.  Hand case: one block-row, two
    identity blocks on block-columns 0 and 1, two streams; y = x[0:16] + x[16:32] with everything on."""
    eye = np.eye(16, dtype=np.int8)
    codes = np.stack([eye, eye])
    col, off = np.array([0, 1], np.int16), np.array([0, 2], np.int32)
    x = np.stack([np.arange(32, dtype=np.float32), 100 + np.arange(32, dtype=np.float32)])
    one = np.float32(1.0)
    full = O.mortar_gemv(x, codes, one, col, off)
    assert np.array_equal(full, x[:, :16] + x[:, 16:])
    cact = np.array([[1, 0], [0, 1]], np.int32)                       # stream 0 keeps column 0, stream 1 keeps column 1
    y = O.mortar_gemv(x, codes, one, col, off, col_act=cact)
    assert np.array_equal(y[0], x[0, :16]) and np.array_equal(y[1], x[1, 16:])
    ract = np.array([[0], [1]], np.int32)                             # the row is off for stream 0 only
    y = O.mortar_gemv(x, codes, one, col, off, row_act=ract)
    assert not y[0].any() and np.array_equal(y[1], full[1])
    y = O.mortar_gemv(x, codes, one, col, off, row_act=ract, col_act=cact)
    assert not y[0].any() and np.array_equal(y[1], x[1, 16:])
    # all flags on == no flags; any non-zero value counts as on
    m = make_mat(5, 8, 0.4, 44)
    xr = xbf(3, 128, 45)
    a = O.mortar_gemv(xr, m["codes"], m["scales"], m["col_idx"], m["offsets"])
    b = O.mortar_gemv(xr, m["codes"], m["scales"], m["col_idx"], m["offsets"], row_act=np.full((3, 5), 7), col_act=np.full((3, 8), -1))
    assert np.array_equal(a, b)
    # against the dense form: flags are a row mask on the output and a column mask on the input, per stream
    rng = np.random.default_rng(46)
    ra, ca = rng.integers(0, 2, (3, 5)), rng.integers(0, 2, (3, 8))
    got = O.mortar_gemv(xr, m["codes"], m["scales"], m["col_idx"], m["offsets"], row_act=ra, col_act=ca)
    W = O.to_dense(m["codes"].astype(np.float64) * m["scales"].astype(np.float64)[:, None, None], m["row_idx"], m["col_idx"], m["shape"])
    want = ((xr.astype(np.float64) * np.repeat(ca, 16, axis=1)) @ W.T) * np.repeat(ra, 16, axis=1)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


# ---- ReMoE ---------------------------------------------------------------------------------------------

def brute_remoe(logits, k):
    out = []
    for row in logits:
        n = len(row)
        if k < n:
            # k-th largest VALUE by counting: smallest v in row with #(row > v) < k
            cands = [v for v in row if (row > v).sum() < k <= (row >= v).sum()]
            kth = cands[0]
            out.append(row > kth)
        else:
            out.append(row > 0)
    return np.array(out)


def test_remoe_brute_force_incl_ties():
    rng = np.random.default_rng(50)
    for n, k in ((8, 3), (16, 8), (6, 1), (5, 5), (7, 6)):
        lg = rng.integers(-3, 4, size=(200, n)).astype(np.float32)            # many ties
        lg[0, :] = 1.0                                                        # all equal -> nothing strictly above
        gates, act = O.remoe_gates(lg, k)
        assert np.array_equal(act, brute_remoe(lg, k))
        gc, ac = c_oracle.remoe_gates(lg, k)
        assert np.array_equal(ac, act) and np.allclose(gc, gates, rtol=1e-6)
        if k < n:
            assert (act.sum(1) <= k - 1).all() and not act[0].any()           # the k-th itself is inactive
        assert (gates >= 0).all()
        on = act.any(1)
        assert np.allclose(gates[on].sum(1), k, rtol=1e-5)                     # normalised to sum k
        assert (gates[~on] == 0).all()


def test_remoe_gate_sum_clamp_known_answer():
    """routing.py:253: the sum of the thresholded logits is clamped at 1e-6 before the division.  One entry sits one
    fp32 ulp above the k-th largest: g0 = (2^-23, 0, 0, 0), sum = 1.19e-7 < 1e-6, so gates = 2^-23 * (2 / 1e-6) =
    0.23841858 (without the clamp: 2.0; with a clamp at 1e-3: 2.38e-4)."""
    import torch
    lg = np.array([[1.0 + 2.0 ** -23, 1.0, 0.0, -1.0]], np.float32)
    gates, act = O.remoe_gates(lg, 2)
    assert act.tolist() == [[True, False, False, False]]
    np.testing.assert_allclose(gates[0], [0.23841858, 0.0, 0.0, 0.0], rtol=1e-6, atol=0)
    gc, ac = c_oracle.remoe_gates(lg, 2)
    np.testing.assert_allclose(gc[0], [0.23841858, 0.0, 0.0, 0.0], rtol=1e-6, atol=0)
    # the same steps written with the library's own ops (topk / relu / clamp), fp32
    t = torch.from_numpy(lg)
    g0 = torch.relu(t - torch.topk(t, 2, dim=-1).values[:, -1:])
    want = g0 * (2.0 / g0.sum(dim=-1, keepdim=True).clamp(min=1e-6))
    assert np.array_equal(gates, want.numpy())
    # a sum just above the clamp is not clamped: normalised to k
    lg2 = np.array([[1.0 + 2.0 ** -19, 1.0, 0.0, -1.0]], np.float32)        # g0 = 1.9e-6 > 1e-6
    np.testing.assert_allclose(O.remoe_gates(lg2, 2)[0][0], [2.0, 0, 0, 0], rtol=1e-6)


def test_router_logits_against_library_routines():
    """Steps 1-4 of the router reduce to library routines: torch's linear, layer_norm and matmul in float64, and the
    reference's broadcast-add / wrap indexing (routing.py:205-230) written with torch indexing."""
    import torch
    rng = np.random.default_rng(52)
    for d, nsk, n in ((64, 4, 16), (48, 3, 20), (32, 2, 4), (64, 5, 20), (32, 19, 352)):
        x = rng.standard_normal((5, d)); wq = rng.standard_normal((d, d)) / np.sqrt(d); it = rng.standard_normal(d) * 0.1
        lw = 1 + 0.1 * rng.standard_normal(d); lb = 0.1 * rng.standard_normal(d)
        ka = rng.standard_normal((nsk, d // 2)); kb = rng.standard_normal((nsk, d // 2)); bias = rng.standard_normal(n)
        got = O.router_logits(x, wq, it, lw, lb, 1e-5, ka, kb, bias)
        t = lambda a: torch.from_numpy(np.asarray(a, np.float64))
        q = torch.nn.functional.layer_norm(torch.nn.functional.linear(t(x), t(wq)) + t(it), (d,), t(lw), t(lb), 1e-5)
        sa, sb = q[:, :d // 2] @ t(ka).T, q[:, d // 2:] @ t(kb).T
        ps = (sa.unsqueeze(2) + sb.unsqueeze(1)).reshape(5, nsk * nsk)
        if nsk * nsk > n:                    # routing.py:212-222: topk over the products, values in descending order
            want = ps.topk(n, dim=-1).values + t(bias).unsqueeze(0)
            assert (np.diff(got - bias, axis=1) <= 0).all()
        else:
            want = ps[:, torch.arange(n) % (nsk * nsk)] + t(bias).unsqueeze(0)
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-12)
        assert np.allclose(O.router_logits(x, wq, None, lw, lb, 1e-5, ka, kb, bias),
                           O.router_logits(x, wq, np.zeros(d), lw, lb, 1e-5, ka, kb, bias))


def test_remoe_distinct_logits_count():
    lg = np.random.default_rng(51).standard_normal((64, 352)).astype(np.float32)
    gates, act = O.remoe_gates(lg, 88)
    assert (act.sum(1) == 87).all()
    top = np.argsort(-lg, axis=1)[:, :87]
    assert all(set(np.nonzero(act[i])[0]) == set(top[i]) for i in range(64))


def test_route_flags_closed_form():
    gates = np.zeros((2, 4), np.float32); gates[0, 1] = 0.5; gates[1, 3] = 2.0   # d_ff 128, 4 clusters of 32
    ract, cact = O.route_flags(gates, 128, 16)
    assert cact.tolist() == [[0, 0, 1, 1, 0, 0, 0, 0], [0, 0, 0, 0, 0, 0, 1, 1]]
    assert ract.tolist() == [c + c for c in cact.tolist()]
    # clusters of 8: block r spans clusters lo = 2r and hi = 2r + 1 (engine.py:384-413); either side alone turns it on
    g_hi = np.zeros((1, 16), np.float32); g_hi[0, 3] = 1.0                       # hi side of block 1 only
    assert O.route_flags(g_hi, 128, 16)[1].tolist() == [[0, 1, 0, 0, 0, 0, 0, 0]]
    g_lo = np.zeros((1, 16), np.float32); g_lo[0, 2] = 1.0                       # lo side of block 1 only
    assert O.route_flags(g_lo, 128, 16)[1].tolist() == [[0, 1, 0, 0, 0, 0, 0, 0]]
    g_lo[0, 2] = 0.0; g_lo[0, 14] = 0.25                                         # lo side of the last block
    rl, cl = O.route_flags(g_lo, 128, 16)
    assert cl.tolist() == [[0, 0, 0, 0, 0, 0, 0, 1]] and rl.tolist() == [[0] * 7 + [1] + [0] * 7 + [1]]
    # clusters of 24 over d_ff 96 (not a multiple of the block): block 1 = features 16..31 straddles clusters 0 | 1,
    # block 4 = features 64..79 straddles 2 | 3
    g24 = np.zeros((1, 4), np.float32); g24[0, 0] = 1.0
    assert O.route_flags(g24, 96, 16)[1].tolist() == [[1, 1, 0, 0, 0, 0]]
    g24[0, 0] = 0.0; g24[0, 3] = 1.0
    assert O.route_flags(g24, 96, 16)[1].tolist() == [[0, 0, 0, 0, 1, 1]]
    # a gate that is not positive does not count (strict > 0), NaN does not either
    gz = np.zeros((1, 16), np.float32); gz[0, 2] = -1.0; gz[0, 5] = np.nan
    assert O.route_flags(gz, 128, 16)[1].sum() == 0


def test_rmsnorm_closed_form():
    # known answers: x = (3, 4) * 1e-3, mean(x^2) = 12.5e-6, eps = 1e-6 -> x * rsqrt(13.5e-6): y = (sqrt(2/3), sqrt(32/27)).
    # eps is as large as 8 % of the mean square here, so eps outside the root, a dropped eps or mean -> sum all miss.
    x = np.array([[3e-3, 4e-3]], dtype=np.float32)
    y = O.rmsnorm(x, None, 1e-6, bf16_out=False)
    np.testing.assert_allclose(y[0], [0.816496580927726, 1.0886621079036347], rtol=2e-6)
    # eps = 1 on x = (3, 4): the same numbers again (rsqrt(12.5 + 1) = rsqrt(13.5)), with eps >> rounding
    y1 = O.rmsnorm(np.array([[3.0, 4.0]], np.float32), None, 1.0, bf16_out=False)
    np.testing.assert_allclose(y1[0], [0.816496580927726, 1.0886621079036347], rtol=1e-6)
    # eps = 0: unit mean square exactly
    y0 = O.rmsnorm(np.array([[3.0, 4.0]], np.float32), None, 0.0, bf16_out=False)
    np.testing.assert_allclose(y0[0], [3 / np.sqrt(12.5), 4 / np.sqrt(12.5)], rtol=1e-6)
    # the weight multiplies after the cast to the activation dtype (attention.py:139-141): bf16(bf16(x r) w)
    # known answer: x = (1, 4), w = 1.375: x r = (0.342997, 1.371989) -> bf16 (0.34375, 1.375) -> * 1.375 =
    # (0.47265625, 1.890625), both exact in bf16.  Rounding once, bf16(x r w), gives (0.47070312, 1.8828125) instead.
    xb = np.array([[1.0, 4.0]], np.float32); w = np.array([1.375, 1.375], np.float32)
    assert O.rmsnorm(xb, w, 1e-6).tolist() == [[0.47265625, 1.890625]]
    r = np.float32(1.0 / np.sqrt(8.5 + 1e-6))
    assert O.bf16_round(xb * r * w).tolist() == [[0.470703125, 1.8828125]]        # the mutant's numbers, for the record
    import torch
    tx = torch.tensor([[1.0, 4.0]], dtype=torch.bfloat16)
    tn = (tx.float() * torch.rsqrt(tx.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16) * torch.tensor(w).to(torch.bfloat16)
    assert tn.float().tolist() == [[0.47265625, 1.890625]]                        # attention.py:139-141 in torch-CPU bf16
    x = xbf(4, 64, 60)
    y = O.rmsnorm(x, None, 1e-6, bf16_out=False)
    assert np.allclose((y.astype(np.float64) ** 2).mean(1), 1.0, atol=1e-4)
    w = np.full(64, 2.0, np.float32)
    assert np.allclose(O.rmsnorm(x, w, bf16_out=False), 2 * y)


def test_hc_post_known_cases():
    rng = np.random.default_rng(81)
    T, n, C = 3, 4, 8
    h, y, term = rng.standard_normal((T, n, C)), rng.standard_normal((T, C)), rng.standard_normal((T, C))
    eye = np.broadcast_to(np.eye(n), (T, n, n))
    assert np.array_equal(O.hc_post(eye, np.zeros((T, n)), h, y), h)                       # identity mixing, y off: the carrier
    assert np.array_equal(O.hc_post(np.zeros((T, n, n)), np.ones((T, n)), h, y), np.broadcast_to(y[:, None], (T, n, C)))
    perm = np.zeros((T, n, n)); perm[:, np.arange(n), (np.arange(n) + 1) % n] = 1.0         # out[i] = h[i + 1]: rows index the OUTPUT
    assert np.array_equal(O.hc_post(perm, np.zeros((T, n)), h, y), np.roll(h, -1, axis=1))
    assert np.allclose(O.hc_post(eye, np.zeros((T, n)), h, y, term), h + term[:, None])    # the term is added to every stream once
    # hand-computed: 2 streams, 1 channel: out0 = 2*10 + 3*20 + 0.5*4 = 82, out1 = -1*10 + 0*20 + 2*4 + 1 = -1
    out = O.hc_post(np.array([[[2.0, 3.0], [-1.0, 0.0]]]), np.array([[0.5, 2.0]]), np.array([[[10.0], [20.0]]]), np.array([[4.0]]))
    assert out.tolist() == [[[82.0], [-2.0]]]
    out = O.hc_post(np.array([[[2.0, 3.0], [-1.0, 0.0]]]), np.array([[0.5, 2.0]]), np.array([[[10.0], [20.0]]]), np.array([[4.0]]), np.array([[1.0]]))
    assert out.tolist() == [[[83.0], [-1.0]]]


def test_bf16_round_matches_torch():
    import torch
    a = np.random.default_rng(70).standard_normal(10000).astype(np.float32) * 1e3
    a[:4] = [0.1, 1.00390625, 1.005859375, -1.00390625]                           # ties-to-even cases
    assert np.array_equal(O.bf16_round(a), torch.from_numpy(a).to(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------------------------------------- committed fixtures

def test_golden_c0_pins_numpy_and_c_oracle():
    """The committed config-0 vectors: both restatements reproduce the stored bf16 output bit for bit."""
    import golden_util as G
    from oracle import c_oracle
    z = G.load("c0_spmm.npz")
    m = G.matrix(z)
    x = O.bf16_from_bits(z["x_bits"])
    assert m["shape"] == (2048, 768) and int(m["offsets"][-1]) == 1536 and z["x_bits"].shape == (64, 768)
    y = O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"], m["shape"])
    assert np.array_equal(O.bf16_bits(y), z["y_bits"])
    yc = c_oracle.bcsr_spmm_bf16(z["x_bits"], m["codes"], m["scales"], m["col_idx"], m["offsets"])
    assert np.array_equal(yc, z["y_bits"])
    # and the stored output is what a dense fp64 matmul of the scattered weight gives (library routine)
    dense = O.to_dense(O.effective_blocks(m["codes"], m["scales"]), m["row_idx"], m["col_idx"], m["shape"])
    assert np.array_equal(O.bf16_bits(x.astype(np.float64) @ dense.astype(np.float64).T), z["y_bits"])


def test_golden_mlp_slice_pins_swiglu_and_gating():
    import golden_util as G
    from oracle import c_oracle
    z = G.load("mlp_slice.npz")
    gu, dn = G.matrix(z, "gate_up_"), G.matrix(z, "down_")
    x = O.bf16_from_bits(z["x_bits"])
    logits = z["logits_bits"].view(np.float32)
    gates, active = O.remoe_gates(logits, 11)
    assert np.array_equal(gates.astype(np.float32).view(np.uint32), z["gates_bits"])
    assert np.array_equal(active.astype(np.uint8), z["active"])
    assert (z["active"].sum(1) <= 10).all()                                    # strict threshold: at most k-1 active
    for g, hk, yk in ((None, "h_bits", "y_bits"), (gates, "h_routed_bits", "y_routed_bits")):
        r = O.swiglu_mlp(x, gu, dn, gates=g)
        assert np.array_equal(O.bf16_bits(r["h"]), z[hk]) and np.array_equal(O.bf16_bits(r["y"]), z[yk])
        _, hc, yc = c_oracle.mlp_bf16(z["x_bits"], gu, dn, 704, gates=None if g is None else g.astype(np.float32))
        assert np.abs(O.bf16_from_bits(hc) - O.bf16_from_bits(z[hk])).max() <= 2 ** -7 * np.abs(O.bf16_from_bits(z[hk])).max()
        assert np.abs(O.bf16_from_bits(yc) - O.bf16_from_bits(z[yk])).max() <= 1e-2 * np.abs(O.bf16_from_bits(z[yk])).max()


# ---- backward products ------------------------------------------------------------------------------

def test_backward_products_against_dense_matmul_and_adjoint_identity():
    """dds_dx and sdd_at_b reduce to dense matmuls (+ gather of the kept blocks), and satisfy the adjoint
    identities of y = x W^T: <dY, y> = <dY W, x> = <dW, blocks of W>.  A transposed operand, a swapped row/column
    index or a block stored transposed fails one of these."""
    rng = np.random.default_rng(5)
    Rb, Cb, M = 5, 7, 37
    mask = rng.random((Rb, Cb)) < 0.5
    mask[np.arange(Rb), rng.integers(0, Cb, Rb)] = True
    r, c = np.nonzero(mask)
    nnz = r.size
    codes = rng.integers(-1, 2, (nnz, 16, 16)).astype(np.int8)
    scales = O.bf16_round(rng.uniform(0.01, 0.1, nnz).astype(np.float32))
    x = O.bf16_round(rng.standard_normal((M, Cb * 16)).astype(np.float32))
    dy = O.bf16_round(rng.standard_normal((M, Rb * 16)).astype(np.float32))
    W = O.to_dense(O.effective_blocks(codes, scales), r, c, (Rb * 16, Cb * 16)).astype(np.float64)
    dx = O.dds_dx(dy, codes, scales, r, c, (Rb * 16, Cb * 16), round_out=False)
    np.testing.assert_allclose(dx, dy.astype(np.float64) @ W, rtol=1e-6, atol=1e-6)
    dw = O.sdd_at_b(dy, x, r, c, round_out=False)
    full = dy.astype(np.float64).T @ x.astype(np.float64)                   # dense dW [out, in]
    for j in range(nnz):
        np.testing.assert_allclose(dw[j], full[r[j] * 16:(r[j] + 1) * 16, c[j] * 16:(c[j] + 1) * 16], rtol=1e-6, atol=1e-5)
    y = x.astype(np.float64) @ W.T
    lhs = float((dy * y).sum())
    np.testing.assert_allclose(float((dx.astype(np.float64) * x).sum()), lhs, rtol=1e-5)
    np.testing.assert_allclose(float((dw.astype(np.float64) * O.effective_blocks(codes, scales)).sum()), lhs, rtol=1e-5)


def test_swiglu_backward_against_central_differences():
    """The unrounded derivative equals the numerical gradient of sum(w * silu(g) * u); the forward equals silu * up."""
    rng = np.random.default_rng(9)
    gu = rng.standard_normal((5, 32)) * 2.0
    w = rng.standard_normal((5, 16))
    f = lambda z: float((w * (z[:, :16] / (1.0 + np.exp(-z[:, :16]))) * z[:, 16:]).sum())
    num = np.zeros_like(gu)
    for i in range(gu.shape[0]):
        for j in range(gu.shape[1]):
            e = np.zeros_like(gu); e[i, j] = 1e-6
            num[i, j] = (f(gu + e) - f(gu - e)) / 2e-6
    got = O.swiglu_backward(gu.astype(np.float64), w, round_out=False)
    np.testing.assert_allclose(got, num, rtol=2e-5, atol=1e-6)      # float32 output of the oracle
    gb = O.bf16_round(gu.astype(np.float32))
    h = O.swiglu(gb)
    np.testing.assert_allclose(h, O.silu(gb[:, :16]) * gb[:, 16:], rtol=2 ** -6, atol=1e-6)


def test_training_fixture_matches_the_oracle():
    """tests/golden/train_slice.npz (ternarisation, forward, dX, dW, SwiGLU and its derivative of one small layer) is
    what the oracle computes today: guards both against drift."""
    import golden_util as G
    z = G.load("train_slice.npz")
    vals = O.bf16_from_bits(z["values_bits"])
    x, dy = O.bf16_from_bits(z["x_bits"]), O.bf16_from_bits(z["dy_bits"])
    q, s = O.ternary_quantize(vals, 0.5)
    assert np.array_equal(q, z["codes"]) and np.float32(s).view(np.uint32) == z["scale_bits"][0]
    qb, sb = O.ternary_quantize_per_block(vals, 0.5)
    assert np.array_equal(qb, z["codes_per_block"]) and np.array_equal(sb.view(np.uint32), z["scale_per_block_bits"])
    shape = tuple(int(v) for v in z["shape"])
    assert np.array_equal(O.bf16_bits(O.bcsr_spmm(x, q, np.float32(s), z["col_idx"], z["offsets"])), z["y_bits"])
    assert np.array_equal(O.bf16_bits(O.dds_dx(dy, q, np.float32(s), z["row_idx"], z["col_idx"], shape)), z["dx_bits"])
    assert np.array_equal(O.bf16_bits(O.sdd_at_b(dy, x, z["row_idx"], z["col_idx"])), z["dw_bits"])
    gu, dh = O.bf16_from_bits(z["gu_bits"]), O.bf16_from_bits(z["dh_bits"])
    assert np.array_equal(O.bf16_bits(O.swiglu(gu)), z["h_bits"])
    assert np.array_equal(O.bf16_bits(O.swiglu_backward(gu, dh)), z["dgu_bits"])


def test_swiglu_family_bit_equal_to_torch_cpu_bf16():
    """The bf16 rounding points of swiglu, swiglu_backward and the gated multiply are those of the eager graph
    (transformer.py:403-427): checked against the library routine itself -- F.silu(gate) * up, its autograd, and
    h.unflatten(-1, (n_clusters, cs)) * gates.to(bf16).unsqueeze(-1) -- in torch-CPU bf16, bit for bit."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(77)
    M, d_ff, ncl = 64, 96, 6
    gu = O.bf16_round((rng.standard_normal((M, 2 * d_ff)) * 3.0).astype(np.float32))
    gu[0, :8] = [0.0, -0.0, 1e-30, -1e-30, 80.0, -80.0, 2.0 ** -120, -20.0]         # saturation / denormal corners
    dh = O.bf16_round(rng.standard_normal((M, d_ff)).astype(np.float32))
    t = torch.from_numpy(gu).to(torch.bfloat16).requires_grad_(True)
    gate, up = t.chunk(2, dim=-1)
    h = F.silu(gate) * up
    assert np.array_equal(O.bf16_bits(O.swiglu(gu)), O.bf16_bits(h.detach().float().numpy()))
    h.backward(torch.from_numpy(dh).to(torch.bfloat16))
    got = O.swiglu_backward(gu, dh)
    want = t.grad.float().numpy()
    # torch's silu backward computes d_gate in fp32 from bf16 inputs with its own operation order; the oracle's
    # float64 calculus rounded once may differ from it by one bf16 ulp in rare entries, never more
    gb, wb = O.bf16_bits(got).astype(np.int64), O.bf16_bits(want).astype(np.int64)
    same = gb == wb
    assert same.mean() > 0.98, same.mean()
    assert np.array_equal(gb[:, d_ff:], wb[:, d_ff:])                                 # d_up = dh * bf16(silu(g)): exact
    assert (np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-30).all()
    # gated multiply: gates cast to bf16 first, product rounded to bf16
    gates = (rng.random((M, ncl)) * 4).astype(np.float32); gates[:, 2] = 0.0
    hb = h.detach()
    hg = (hb.unflatten(-1, (ncl, d_ff // ncl)) * torch.from_numpy(gates).to(hb.dtype).unsqueeze(-1)).flatten(-2)
    x = O.bf16_round(rng.standard_normal((M, 32)).astype(np.float32))
    eye_gu = dict(codes=np.zeros((0, 16, 16), np.int8))                              # not used: call the pieces directly
    hn = O.bf16_round(O.bf16_round(O.silu(gu[:, :d_ff])) * gu[:, d_ff:])              # as swiglu_mlp forms h
    gbf = O.bf16_round(gates)
    mine = O.bf16_round(hn.reshape(-1, ncl, d_ff // ncl) * gbf[:, :, None]).reshape(-1, d_ff)
    assert np.array_equal(O.bf16_bits(mine), O.bf16_bits(hg.float().numpy()))
    assert np.array_equal(O.bf16_bits(hn), O.bf16_bits(hb.float().numpy()))          # swiglu_mlp's fp32 silu == swiglu's


def test_swiglu_mlp_gating_is_the_torch_expression():
    """swiglu_mlp end to end on a tiny carved pair, against torch-CPU bf16 ops for everything after gate_up
    (F.silu * up, cluster gates cast to bf16) and the dense float64 product for the matrices."""
    import torch
    import torch.nn.functional as F
    gu, dn = make_mat(2 * 6, 4, 0.5, 33), make_mat(4, 6, 0.5, 34)
    x = xbf(9, 64, 35)
    gates = (np.random.default_rng(36).random((9, 3)) * 3).astype(np.float32); gates[::2, 1] = 0
    r = O.swiglu_mlp(x, gu, dn, gates=gates)
    t = torch.from_numpy(r["gu"]).to(torch.bfloat16)
    g, u = t.chunk(2, dim=-1)
    h = F.silu(g) * u
    h = (h.unflatten(-1, (3, 32)) * torch.from_numpy(gates).to(h.dtype).unsqueeze(-1)).flatten(-2)
    assert np.array_equal(O.bf16_bits(r["h"]), O.bf16_bits(h.float().numpy()))
