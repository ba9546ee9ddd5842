"""CPU oracle for the MORTAR sparse-MLP path (TEST INFRASTRUCTURE, not product code).

Plain numpy restatement of the reference's algorithm for the carved block-sparse
ternary MLP.  Only tests, the smoke check and the CPU-baseline leg of the benchmark
may import this module; the product package never does.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  How each function is pinned (no reference import is needed):

  carve / to_dense         closed form + brute-force scatter round trip
  ternary_quantize         closed form + "all non-zero magnitudes equal one scale"
  pack/unpack_ternary      exhaustive over all 256 byte values
  pack_strips / work_list  closed form + partition invariants
  bcsr_spmm                reduces to dense scatter + float64 matmul; special cases
  dds_dx / sdd_at_b        (backward) reduce to dense float64 matmuls + a gather of the
                           kept blocks; the adjoint identity <dY, x W^T> = <dY W, x> = <dW, W>
  swiglu_mlp               textbook x*sigmoid(x) + the above
  swiglu / swiglu_backward the same closed form; the derivative by central differences
  remoe_gates              brute force on tiny inputs incl. ties; invariants
  route_flags              closed form
  rmsnorm                  closed form
  hc_post                  special cases with known results (identity mixing, pure pass-through of y, a
                           permutation of the streams) + a hand-computed 2-stream case
  transpose_meta           order of blocks *inside one block-column* depends on the
                           reference's unstable argsort: PARITY UNPINNED for that
                           order (backward-only metadata, not on the forward path)

bfloat16 is carried as float32 arrays holding bf16-representable values (see
``bf16_round``) or as uint16 bit patterns (``bf16_bits``).
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------- bf16


def bf16_bits(a) -> np.ndarray:
    """float32 -> bf16 bit pattern (uint16), round-to-nearest-even (torch .to(bfloat16))."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    if nan.any():
        r = np.where(nan, np.uint16(0x7FC0), r)
    return r


def bf16_from_bits(b) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def bf16_round(a) -> np.ndarray:
    """float32 -> nearest bf16 value, returned as float32."""
    return bf16_from_bits(bf16_bits(a))


# --------------------------------------------------------------------------- carve


def carve(w: np.ndarray, block_mask: np.ndarray, blocking: int = 16) -> dict:
    """Dense masked [out, in] -> BCSR.  morph/model/layers/block_sparse.py:810-907.

    block_mask [Rb, Cb] bool.  Row-major nonzero() order (sorted by row then column,
    :874-878); int16 row/column indices, int32 offsets = [0, cumsum(row_nnz)]
    (:877-883); data[j, lr, c] = W[row_j*blk+lr, col_j*blk+c] (:885-888).
    """
    out_f, in_f = w.shape
    if out_f % blocking or in_f % blocking:
        raise ValueError(f"carve: [{out_f},{in_f}] not divisible by blocking {blocking}")
    Rb, Cb = out_f // blocking, in_f // blocking
    bm = np.asarray(block_mask, dtype=bool)
    assert bm.shape == (Rb, Cb)
    if not bm.any(axis=1).all():
        raise RuntimeError("carve: a block-row has zero kept blocks")     # :871-872
    idx = np.argwhere(bm)                                                  # row-major
    rows = idx[:, 0].astype(np.int16)
    cols = idx[:, 1].astype(np.int16)
    offsets = np.concatenate([[0], np.cumsum(bm.sum(axis=1))]).astype(np.int32)
    blocks = w.reshape(Rb, blocking, Cb, blocking).transpose(0, 2, 1, 3)
    data = np.ascontiguousarray(blocks[idx[:, 0], idx[:, 1]])
    ct, ot, bt = transpose_meta((out_f, in_f), blocking, rows, cols)
    return dict(mortar_data=data, mortar_row_indices=rows, mortar_column_indices=cols,
                mortar_offsets=offsets, mortar_column_indices_t=ct, mortar_offsets_t=ot,
                mortar_block_offsets_t=bt)


def transpose_meta(size, blocking, row_indices, column_indices):
    """morph/sparse/stk/matrix.py:107-125.  A STABLE sort is used here; the reference's
    default argsort leaves the order of blocks within one block-column unspecified."""
    block_columns = size[1] // blocking
    gather = np.argsort(column_indices.astype(np.int64), kind="stable")
    column_indices_t = row_indices[gather].astype(np.int16)
    block_offsets_t = gather.astype(np.int32)
    nnz_per_col = np.bincount(column_indices.astype(np.int64), minlength=block_columns)
    offsets_t = np.concatenate([[0], np.cumsum(nnz_per_col)]).astype(np.int32)
    return column_indices_t, offsets_t, block_offsets_t


def to_dense(data, row_indices, column_indices, shape, blocking: int = 16) -> np.ndarray:
    """Scatter [nnz, blk, blk] blocks into a dense [out, in] matrix.
    morph/sparse/stk/ops/matrix_ops.py:37-49; morph/inference/engine.py:74-84."""
    out_f, in_f = shape
    W = np.zeros((out_f // blocking, blocking, in_f // blocking, blocking), dtype=data.dtype)
    W[row_indices.astype(np.int64), :, column_indices.astype(np.int64)] = data
    return W.reshape(out_f, in_f)


# --------------------------------------------------------------------------- ternary


def ternary_quantize(w: np.ndarray, threshold: float = 0.5):
    """Per-tensor symmetric ternary.  morph/inference/deploy_quant.py:81-95;
    block_sparse.py:909-919.  scale = mean|w| clamped at 1e-8; q = sign(w/s)*(|w/s| > thr)."""
    wf = np.asarray(w, dtype=np.float32)
    scale = np.float32(max(np.float32(np.abs(wf).mean(dtype=np.float32)), np.float32(1e-8)))
    wn = wf / scale
    q = (np.sign(wn) * (np.abs(wn) > np.float32(threshold))).astype(np.int8)
    return q, scale


def ternary_quantize_per_block(w: np.ndarray, threshold: float = 0.5):
    """Per-16x16-tile form of the same rule: scale per block = mean|w| clamped at 1e-6.
    block_sparse.py:341-349,393-401.  w [nnz, blk, blk] -> (codes int8, scale [nnz] fp32)."""
    wf = np.asarray(w, dtype=np.float32)
    scale = np.maximum(np.abs(wf).mean(axis=(1, 2), dtype=np.float32), np.float32(1e-6)).astype(np.float32)
    wn = wf / scale[:, None, None]
    q = (np.sign(wn) * (np.abs(wn) > np.float32(threshold))).astype(np.int8)
    return q, scale


def pack_ternary_codes(q: np.ndarray) -> np.ndarray:
    """2-bit pack, 4 codes/byte, u = code+1, little-endian in the byte, zero padded to x4.
    morph/inference/deploy_quant.py:56-71."""
    flat = np.asarray(q).reshape(-1)
    pad = (-flat.size) % 4
    u = (flat.astype(np.int16) + 1).astype(np.uint8)
    if pad:
        u = np.concatenate([u, np.zeros(pad, dtype=np.uint8)])
    u = u.reshape(-1, 4)
    return (u[:, 0] | (u[:, 1] << 2) | (u[:, 2] << 4) | (u[:, 3] << 6)).astype(np.uint8)


def unpack_ternary(packed: np.ndarray, numel: int) -> np.ndarray:
    """Inverse of pack_ternary_codes -> int8 in {-1,0,+1} (3 -> +2 never produced).
    morph/inference/deploy_quant.py:74-78."""
    p = np.asarray(packed, dtype=np.uint8)
    u = (p[:, None] >> np.array([0, 2, 4, 6], dtype=np.uint8)) & 3
    return (u.reshape(-1)[:numel].astype(np.int8) - 1)


def pack_strips(codes: np.ndarray) -> np.ndarray:
    """Engine strip re-pack: byte (j, lr, b) holds columns {b, blk/4+b, 2blk/4+b, 3blk/4+b}.
    morph/kernels/triton/fused_decode_step.py:1465-1478."""
    nnz, blk, _ = codes.shape
    u = (codes.astype(np.int16) + 1).astype(np.uint8).reshape(nnz, blk, 4, blk // 4)
    return (u[:, :, 0] | (u[:, :, 1] << 2) | (u[:, :, 2] << 4) | (u[:, :, 3] << 6)).astype(np.uint8)


def work_list(offsets: np.ndarray, cb: int = 4):
    """Balanced decode work list: one entry per <=cb consecutive blocks of one row.
    fused_decode_step.py:1481-1497.  Returns (ent [3,E] int32 row|j0|slot, nspl_max, cnts [R])."""
    rows, j0s, slots = [], [], []
    R = len(offsets) - 1
    nspl_max = 0
    for r in range(R):
        lo, hi = int(offsets[r]), int(offsets[r + 1])
        nch = -(-(hi - lo) // cb)
        nspl_max = max(nspl_max, nch)
        for s in range(nch):
            rows.append(r); j0s.append(lo + s * cb); slots.append(s)
    ent = np.array([rows, j0s, slots], dtype=np.int32).reshape(3, -1)
    cnts = (-(-(offsets[1:] - offsets[:-1]) // cb)).astype(np.int32)
    return ent, nspl_max, cnts


# --------------------------------------------------------------------------- SpMM


def effective_blocks(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """Deploy dequantisation: bf16(code) * bf16(scale) -> exactly +-bf16(scale) or 0.
    morph/inference/deploy_quant.py:367-369 (scale rounded to bf16).  scales scalar or [nnz]."""
    s = bf16_round(np.broadcast_to(np.asarray(scales, dtype=np.float32).reshape(-1), (codes.shape[0],)))
    return codes.astype(np.float32) * s[:, None, None]


def bcsr_spmm(x: np.ndarray, codes: np.ndarray, scales, col_idx: np.ndarray, offsets: np.ndarray,
              round_out: bool = True, acc_dtype=np.float64) -> np.ndarray:
    """y = x @ W_sparse^T, blockwise in CSR order.
    out[m, r*blk+n] = sum_{j in row r} sum_c x[m, col_j*blk+c] * data[j, n, c]
    (morph/sparse/stk/backend/triton_kernels.py:170-230 with trans_B; decode form
    fused_decode_step.py:1335).  x float32 array of bf16-representable values [M, in];
    returns float32 [M, out] rounded to bf16 when round_out (custom_ops.py:49)."""
    M = x.shape[0]
    nnz, blk, _ = codes.shape
    Rb = len(offsets) - 1
    w = effective_blocks(codes, scales).astype(acc_dtype)
    xa = x.astype(acc_dtype)
    y = np.zeros((M, Rb * blk), dtype=acc_dtype)
    for r in range(Rb):
        lo, hi = int(offsets[r]), int(offsets[r + 1])
        if hi == lo:
            continue
        cols = col_idx[lo:hi].astype(np.int64)
        xs = xa.reshape(M, -1, blk)[:, cols, :]                   # [M, n, blk]
        y[:, r * blk:(r + 1) * blk] = np.einsum("mjc,jnc->mn", xs, w[lo:hi], optimize=True)
    y = y.astype(np.float32)
    return bf16_round(y) if round_out else y


def dds_dx(dy: np.ndarray, codes: np.ndarray, scales, row_idx, col_idx, shape, blk: int = 16,
           round_out: bool = True) -> np.ndarray:
    """dX = dY @ W: the dds product with transpose_b=False over the transposed metadata
    (morph/sparse/stk/backend/custom_ops.py:113-119; kernel triton_kernels.py:170-230 without trans_B).
    dy float32 array of bf16-representable values [M, out] -> float32 [M, in], rounded to bf16 when round_out."""
    W = to_dense(effective_blocks(codes, scales), row_idx, col_idx, shape, blk).astype(np.float64)
    dx = (dy.astype(np.float64) @ W).astype(np.float32)
    return bf16_round(dx) if round_out else dx


def sdd_at_b(a: np.ndarray, b: np.ndarray, row_idx, col_idx, blk: int = 16, round_out: bool = True) -> np.ndarray:
    """a^T @ b restricted to the kept blocks: out[j, lr, c] = sum_m a[m, row_j*blk+lr] * b[m, col_j*blk+c]
    (stk_sdd_at_b, morph/sparse/stk/backend/custom_ops.py:78-96; the dW of the carved forward with a = dY, b = x).
    a [M, out], b [M, in] float32 arrays of bf16-representable values -> float32 [nnz, blk, blk]."""
    M = a.shape[0]
    at = a.astype(np.float64).reshape(M, -1, blk)[:, np.asarray(row_idx, dtype=np.int64), :]     # [M, nnz, blk]
    bt = b.astype(np.float64).reshape(M, -1, blk)[:, np.asarray(col_idx, dtype=np.int64), :]
    out = np.einsum("mjl,mjc->jlc", at, bt, optimize=True).astype(np.float32)
    return bf16_round(out) if round_out else out


def dense_linear(x: np.ndarray, codes, scales, row_idx, col_idx, shape, blk=16) -> np.ndarray:
    """The reference's CPU-expressible twin: dense scatter + matmul (float64), unrounded."""
    W = to_dense(effective_blocks(codes, scales), row_idx, col_idx, shape, blk).astype(np.float64)
    return (x.astype(np.float64) @ W.T).astype(np.float32)


def silu(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.float32)
    return (x / (np.float32(1.0) + np.exp(-x, dtype=np.float32))).astype(np.float32)


def swiglu(gu: np.ndarray) -> np.ndarray:
    """h = bf16(bf16(silu(gate)) * up), gate = gu[:, :d_ff], up = gu[:, d_ff:]  (transformer.py:411-413, the bf16
    tensors the eager path materialises).  gu float32 array of bf16-representable values."""
    d_ff = gu.shape[1] // 2
    g, u = gu[:, :d_ff].astype(np.float64), gu[:, d_ff:].astype(np.float64)
    s = bf16_round((g / (1.0 + np.exp(-g))).astype(np.float32)).astype(np.float64)
    return bf16_round((s * u).astype(np.float32))


def swiglu_backward(gu: np.ndarray, dh: np.ndarray, round_out: bool = True) -> np.ndarray:
    """d gu from dh for h = silu(gate) * up: d_up = dh * silu(g); d_gate = dh * up * sig(g) * (1 + g * (1 - sig(g)))
    (what torch autograd derives for transformer.py:411-413).  With round_out the bf16 tensors of that graph are
    rounded where they appear (silu(g), dh * up, the two results); without, plain float64 calculus."""
    d_ff = gu.shape[1] // 2
    g, u, d = gu[:, :d_ff].astype(np.float64), gu[:, d_ff:].astype(np.float64), dh.astype(np.float64)
    sg = 1.0 / (1.0 + np.exp(-g))
    r = (lambda a: bf16_round(a.astype(np.float32)).astype(np.float64)) if round_out else (lambda a: a)
    d_up = r(d * r(g * sg))
    d_gate = r(r(d * u) * (sg * (1.0 + g * (1.0 - sg))))
    return np.concatenate([d_gate, d_up], axis=1).astype(np.float32)


def swiglu_mlp(x, gate_up: dict, down: dict, gates: np.ndarray | None = None,
               n_clusters: int | None = None) -> dict:
    """_SwiGLUMortar.forward, morph/model/transformer.py:402-431, with every intermediate
    rounded to the activation dtype (bf16) where the reference materialises a tensor:
    gu (bf16) -> silu(gate) (bf16) -> *up (bf16) -> [* gates.to(bf16) per cluster (bf16)] -> down (bf16).
    gate_up/down dicts: codes, scales, col_idx, offsets.  gates [M, n_clusters] fp32 or None."""
    gu = bcsr_spmm(x, gate_up["codes"], gate_up["scales"], gate_up["col_idx"], gate_up["offsets"])
    d_ff = gu.shape[1] // 2
    g, u = gu[:, :d_ff], gu[:, d_ff:]
    h = bf16_round(bf16_round(silu(g)) * u)
    if gates is not None:
        ncl = gates.shape[1] if n_clusters is None else n_clusters
        assert d_ff % ncl == 0
        cs = d_ff // ncl
        gb = bf16_round(gates.astype(np.float32))
        h = bf16_round(h.reshape(-1, ncl, cs) * gb[:, :, None]).reshape(-1, d_ff)
    y = bcsr_spmm(h, down["codes"], down["scales"], down["col_idx"], down["offsets"])
    return dict(gu=gu, h=h, y=y)


# --------------------------------------------------------------------------- decode (fp32 engine form)


def mortar_gemv(x: np.ndarray, codes, scales, col_idx, offsets, row_act=None, col_act=None) -> np.ndarray:
    """Decode GEMV in the engine's arithmetic: fp32 activations, exact +-x/0 products,
    scale applied to each block's partial sum (per-block generalisation of the scalar
    scale-after-sum, fused_decode_step.py:1335,1441-1459).  Returns fp32 [B, O].
    row_act [B, Rb] / col_act [B, Cb] (optional) are the per-stream gather flags of the kernel: the sum of output
    block-row r is zero for stream b when row_act[b, r] == 0 (the CTA stores a zero partial and returns,
    fused_decode_step.py:1378-1381), and a block whose input block-column c has col_act[b, c] == 0 contributes nothing to
    stream b (:1387-1393).  Each stream reads only its own flags."""
    B = x.shape[0]
    nnz, blk, _ = codes.shape
    Rb = len(offsets) - 1
    s = np.broadcast_to(np.asarray(scales, dtype=np.float32).reshape(-1), (nnz,)).astype(np.float64)
    xa = x.astype(np.float64).reshape(B, -1, blk)
    y = np.zeros((B, Rb * blk), dtype=np.float64)
    for r in range(Rb):
        lo, hi = int(offsets[r]), int(offsets[r + 1])
        cols = col_idx[lo:hi].astype(np.int64)
        part = np.einsum("bjc,jnc->bjn", xa[:, cols, :], codes[lo:hi].astype(np.float64))
        if col_act is not None:
            part = part * (np.asarray(col_act)[:, cols] != 0)[:, :, None]
        row = (part * s[lo:hi][None, :, None]).sum(axis=1)
        if row_act is not None:
            row = row * (np.asarray(row_act)[:, r] != 0)[:, None]
        y[:, r * blk:(r + 1) * blk] = row
    return y.astype(np.float32)


# --------------------------------------------------------------------------- ReMoE


def kth_largest(logits: np.ndarray, k: int) -> np.ndarray:
    """Value of the k-th largest entry per row (torch.topk(...).values[:, -1])."""
    return np.sort(logits, axis=-1)[:, ::-1][:, k - 1]


def router_logits(x, wq, iter_vec, ln_w, ln_b, ln_eps, ka, kb, bias) -> np.ndarray:
    """TileRouter.forward steps 1-4, morph/model/routing.py:181-230 (float64 here): q = LayerNorm(x Wq^T + iter_vec);
    sa = q[:, :d/2] Ka^T, sb = q[:, d/2:] Kb^T; product scores ps[a*nsk + b] = sa[a] + sb[b]; group logits = ps + bias
    when nsk^2 == n (:205-211), ps[g mod nsk^2] + bias when nsk^2 < n (:227-230).  LayerNorm uses the biased variance
    (torch.nn.LayerNorm); with nsk^2 > n the group logits are the n largest product scores, descending (:212-222)."""
    x = np.asarray(x, np.float64)
    qv = x @ np.asarray(wq, np.float64).T
    if iter_vec is not None:
        qv = qv + np.asarray(iter_vec, np.float64)
    mean = qv.mean(axis=-1, keepdims=True)
    var = ((qv - mean) ** 2).mean(axis=-1, keepdims=True)
    q = (qv - mean) / np.sqrt(var + ln_eps) * np.asarray(ln_w, np.float64) + np.asarray(ln_b, np.float64)
    d2 = q.shape[1] // 2
    sa = q[:, :d2] @ np.asarray(ka, np.float64).T
    sb = q[:, d2:] @ np.asarray(kb, np.float64).T
    nsk = sa.shape[1]
    ps = (sa[:, :, None] + sb[:, None, :]).reshape(x.shape[0], nsk * nsk)
    n = np.asarray(bias).size
    if nsk * nsk > n:          # :212-222: the n largest product scores in descending order (torch.topk(...).values)
        return np.sort(ps, axis=1)[:, ::-1][:, :n] + np.asarray(bias, np.float64)
    return ps[:, np.arange(n) % (nsk * nsk)] + np.asarray(bias, np.float64)


def remoe_gates(logits: np.ndarray, k: int):
    """TileRouter.forward steps 5-8, morph/model/routing.py:232-284:
    kth = k-th largest value; g0 = relu(logits - kth); gates = g0 * (k / clamp(sum g0, 1e-6));
    active = gates > 0.  The k-th entry itself gets gate 0 and is inactive (strict >),
    morph/kernels/triton/fused_router.py:88-97.  Threshold only when k < n (:236)."""
    lg = np.asarray(logits, dtype=np.float32)
    n = lg.shape[-1]
    if k < n:
        kth = kth_largest(lg, k)[:, None]
        g0 = np.maximum(lg - kth, np.float32(0)).astype(np.float32)
    else:
        g0 = np.maximum(lg, np.float32(0)).astype(np.float32)
    gsum = np.maximum(g0.sum(axis=-1, keepdims=True, dtype=np.float32), np.float32(1e-6))
    gates = (g0 * (np.float32(k) / gsum)).astype(np.float32)
    return gates, gates > 0


def route_flags(gates: np.ndarray, d_ff: int, blk: int = 16):
    """Per-stream gather flags.  fused_decode_step.py:1883-1927 with the span tables of
    morph/inference/engine.py:384-413: lo=(r*blk)//cls, hi=(r*blk+blk-1)//cls;
    row flags cover gate_up's 2*d_ff/blk output block-rows (gate half then up half share
    the map), col flags cover down's d_ff/blk input block-columns.  int32 [B, NR], [B, NC]."""
    ncls = gates.shape[1]
    assert d_ff % ncls == 0
    cls = d_ff // ncls
    r = np.arange(d_ff // blk)
    lo = (r * blk) // cls
    hi = (r * blk + blk - 1) // cls
    col = ((gates[:, lo] > 0) | (gates[:, hi] > 0)).astype(np.int32)
    return np.concatenate([col, col], axis=1), col


# --------------------------------------------------------------------------- hyper-connection POST


def hc_post(hres: np.ndarray, hpost: np.ndarray, h: np.ndarray, y: np.ndarray, term: np.ndarray | None = None) -> np.ndarray:
    """out[t, i, c] = sum_j Hres[t, i, j] * h[t, j, c] + Hpost_row[t, i] * y[t, c] (+ term[t, c]): the POST write of the
    hyper-connection residual around the MLP (morph/kernels/triton/fused_hyper_connection.py:927-970; wide form
    morph/kernels/triton/fused_decode_step.py:1725-1739; call site morph/inference/engine.py:996-1001, 1052-1060).
    hres [T, n, n], hpost [T, n], h [T, n, C], y [T, C], term [T, C] or None -> float64 [T, n, C], unrounded."""
    out = np.einsum("tij,tjc->tic", hres.astype(np.float64), h.astype(np.float64))
    out = out + hpost.astype(np.float64)[:, :, None] * y.astype(np.float64)[:, None, :]
    if term is not None:
        out = out + term.astype(np.float64)[:, None, :]
    return out


# --------------------------------------------------------------------------- RMSNorm


def rmsnorm(x: np.ndarray, weight: np.ndarray | None = None, eps: float = 1e-6, bf16_out: bool = True):
    """x.float() * rsqrt(mean(x^2) + eps) -> cast to x dtype -> * weight.
    morph/model/attention.py:133-141."""
    xf = x.astype(np.float32)
    norm = np.float32(1.0) / np.sqrt(np.mean(xf * xf, axis=-1, keepdims=True, dtype=np.float32) + np.float32(eps))
    y = (xf * norm).astype(np.float32)
    if bf16_out:
        y = bf16_round(y)
    if weight is not None:
        y = y * weight.astype(np.float32)
        if bf16_out:
            y = bf16_round(y)
    return y
