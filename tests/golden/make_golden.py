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


if __name__ == "__main__":
    c0()
    mlp_slice()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
