"""Loaders of the committed fixtures under tests/golden (see tests/golden/make_golden.py)."""
import os

import numpy as np

from oracle import mortar_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def matrix(z, prefix=""):
    """The carve-layout dict (codes int8 [nnz,16,16], scales fp32, col_idx, offsets, row_idx, shape) of a fixture."""
    offsets = z[prefix + "offsets"].astype(np.int32)
    nnz = int(offsets[-1])
    codes = O.unpack_ternary(z[prefix + "packed"], nnz * 256).reshape(nnz, 16, 16).astype(np.int8)
    shape = tuple(int(v) for v in z[prefix + "shape"])
    return dict(codes=codes, scales=z[prefix + "scale_bits"].view(np.float32), col_idx=z[prefix + "col_idx"].astype(np.int16),
                offsets=offsets, row_idx=np.repeat(np.arange(len(offsets) - 1), np.diff(offsets)).astype(np.int16), shape=shape)


def load(name):
    return np.load(os.path.join(GOLDEN, name))
