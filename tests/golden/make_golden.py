"""Writes the golden fixtures of this directory from the seeded generators and the numpy oracle.

    python tests/golden/make_golden.py

The reference's tests hold no numeric vectors for this path, so these fixtures are the build's own: inputs are
drawn by mortar_amd.synth (documented draw order, fixed seeds) and expected outputs are computed by the
plain numpy oracle (float64 accumulation).  They pin the oracle and the C restatement against drift and give the
GPU tests data that does not depend on regenerating inputs.  All arrays are stored as integers (bf16 as uint16
bit patterns, fp32 via their bit patterns) so that no text round trip can change a value.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from mortar_amd import synth  # noqa: E402
from oracle import mortar_oracle as O  # noqa: E402


def c0():
    """benchmark config 0 whole: x [64, 768] bf16, W [2048, 768] at 25 % block density, ternary (.3/.4/.3),
    per-block scale U(.01, .1)."""
    m = synth.synth_matrix(2048, 768, 0.25, seed=100)
    x = synth.synth_x(64, 768, seed=101)
    y = O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"], m["shape"])
    np.savez_compressed(os.path.join(HERE, "c0_spmm.npz"),
                        packed=O.pack_ternary_codes(m["codes"]), scale_bits=m["scales"].view(np.uint32),
                        col_idx=m["col_idx"], offsets=m["offsets"], shape=np.array(m["shape"], np.int64),
                        x_bits=O.bf16_bits(x), y_bits=O.bf16_bits(y))


def mlp_slice():
    """A slice of configs 2/3: d_model 256, d_ff 704 (44 block-rows), Zipf rows, 8 tokens, 44 clusters, k = 11."""
    spec = synth.synth_mlp(256, 16 * 44, 0.25, seed=7, zipf_s=1.2)
    x = synth.synth_x(8, 256, seed=8)
    logits = synth.synth_logits(8, 44, seed=9)
    gates, active = O.remoe_gates(logits, 11)
    out = {}
    for name in ("gate_up", "down"):
        m = spec[name]
        out.update({f"{name}_packed": O.pack_ternary_codes(m["codes"]), f"{name}_scale_bits": m["scales"].view(np.uint32),
                    f"{name}_col_idx": m["col_idx"], f"{name}_offsets": m["offsets"],
                    f"{name}_shape": np.array(m["shape"], np.int64)})
    plain = O.swiglu_mlp(x, spec["gate_up"], spec["down"])
    routed = O.swiglu_mlp(x, spec["gate_up"], spec["down"], gates=gates)
    np.savez_compressed(os.path.join(HERE, "mlp_slice.npz"), x_bits=O.bf16_bits(x), logits_bits=logits.view(np.uint32),
                        gates_bits=gates.astype(np.float32).view(np.uint32), active=active.astype(np.uint8),
                        h_bits=O.bf16_bits(plain["h"]), y_bits=O.bf16_bits(plain["y"]),
                        h_routed_bits=O.bf16_bits(routed["h"]), y_routed_bits=O.bf16_bits(routed["y"]), **out)


def train_slice():
    """One QAT layer's training step: smooth block values (bf16) on a 20 x 12 block topology with Zipf rows, 77 tokens.
    Expected: the ternarisation (codes, per-matrix and per-block scales), y = x W^T, dx = dy W, dW = dy^T x on the
    topology, and the SwiGLU derivative of a 77 x (2 x 96) gate_up output."""
    m = synth.synth_matrix(16 * 20, 16 * 12, 0.3, seed=31, zipf_s=1.2)
    nnz = m["col_idx"].size
    rng = np.random.Generator(np.random.PCG64(77))
    vals = O.bf16_round((rng.standard_normal((nnz, 16, 16), dtype=np.float32) * 0.05).astype(np.float32))
    x, dy = O.bf16_round(synth.synth_x(77, 16 * 12, seed=78)), O.bf16_round(synth.synth_x(77, 16 * 20, seed=79))
    q, s = O.ternary_quantize(vals, 0.5)
    qb, sb = O.ternary_quantize_per_block(vals, 0.5)
    y = O.bcsr_spmm(x, q, np.float32(s), m["col_idx"], m["offsets"])
    dx = O.dds_dx(dy, q, np.float32(s), m["row_idx"], m["col_idx"], m["shape"])
    dw = O.sdd_at_b(dy, x, m["row_idx"], m["col_idx"])
    gu = O.bf16_round(synth.synth_x(77, 192, seed=80) * 2.0)
    dh = O.bf16_round(synth.synth_x(77, 96, seed=81))
    np.savez_compressed(os.path.join(HERE, "train_slice.npz"), col_idx=m["col_idx"], offsets=m["offsets"],
                        row_idx=m["row_idx"], shape=np.array(m["shape"], np.int64), values_bits=O.bf16_bits(vals),
                        codes=q, scale_bits=np.float32(s).reshape(1).view(np.uint32), codes_per_block=qb,
                        scale_per_block_bits=sb.view(np.uint32), x_bits=O.bf16_bits(x), dy_bits=O.bf16_bits(dy),
                        y_bits=O.bf16_bits(y), dx_bits=O.bf16_bits(dx), dw_bits=O.bf16_bits(dw), gu_bits=O.bf16_bits(gu),
                        dh_bits=O.bf16_bits(dh), h_bits=O.bf16_bits(O.swiglu(gu)),
                        dgu_bits=O.bf16_bits(O.swiglu_backward(gu, dh)))


if __name__ == "__main__":
    c0()
    mlp_slice()
    train_slice()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
