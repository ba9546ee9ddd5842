"""ctypes loader for the C oracle (test infrastructure; never imported by the product)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmortar_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "mortar_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmortar_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def bcsr_spmm_bf16(x_bits, codes, scale, col_idx, offsets):
    """x_bits uint16 [M,K] -> y bits uint16 [M, Rb*16]."""
    M, K = x_bits.shape
    Rb = len(offsets) - 1
    nnz = codes.shape[0]
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scale = np.ascontiguousarray(np.broadcast_to(np.asarray(scale, np.float32).reshape(-1), (nnz,)))
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int16)
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    y = np.empty((M, Rb * 16), dtype=np.uint16)
    lib().oracle_bcsr_spmm_bf16(_p(x_bits), M, K, _p(codes), _p(scale), _p(col_idx), _p(offsets), Rb, _p(y))
    return y


def mlp_bf16(x_bits, gu, dn, d_ff, gates=None):
    """gu/dn dicts with codes, scales, col_idx, offsets.  Returns (gu_bits, h_bits, y_bits)."""
    M, d_model = x_bits.shape
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)

    def prep(d):
        nnz = d["codes"].shape[0]
        return (np.ascontiguousarray(d["codes"], np.int8),
                np.ascontiguousarray(np.broadcast_to(np.asarray(d["scales"], np.float32).reshape(-1), (nnz,))),
                np.ascontiguousarray(d["col_idx"], np.int16), np.ascontiguousarray(d["offsets"], np.int32))
    a, b = prep(gu), prep(dn)
    gub = np.empty((M, 2 * d_ff), np.uint16)
    h = np.empty((M, d_ff), np.uint16)
    y = np.empty((M, d_model), np.uint16)
    if gates is not None:
        gates = np.ascontiguousarray(gates, np.float32)
        gp, ncl = _p(gates), gates.shape[1]
    else:
        gp, ncl = None, 0
    lib().oracle_mlp_bf16(_p(x_bits), M, d_model, d_ff, _p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]),
                          _p(b[0]), _p(b[1]), _p(b[2]), _p(b[3]), gp, ncl, _p(gub), _p(h), _p(y))
    return gub, h, y


def remoe_gates(logits, k):
    logits = np.ascontiguousarray(logits, np.float32)
    M, n = logits.shape
    gates = np.empty((M, n), np.float32)
    act = np.empty((M, n), np.uint8)
    lib().oracle_remoe_gates(_p(logits), M, n, int(k), _p(gates), _p(act))
    return gates, act.astype(bool)


def num_threads() -> int:
    return int(lib().oracle_num_threads())
