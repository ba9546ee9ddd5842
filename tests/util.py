"""Shared helpers for the parity tests."""
import numpy as np
import torch

from oracle import mortar_oracle as O


def to_dev(x_f32: np.ndarray, dev) -> torch.Tensor:
    return torch.from_numpy(x_f32).to(torch.bfloat16).to(dev)


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def assert_close_bf16(got: np.ndarray, ref: np.ndarray, what: str = "", ulps: float = 2.0, max_rel: float = 1e-2):
    """The bar for bf16 outputs: max |got - ref| <= 1e-2 * max |ref| (max relative error against the
    fp32/64-accumulated oracle), and elementwise within `ulps` bf16 ulps of the reference magnitude plus a
    small absolute floor that covers cancellation in the sum."""
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), what
    scale = np.abs(ref).max() + 1e-30
    err = np.abs(got - ref)
    assert err.max() <= max_rel * scale, f"{what}: max rel err {err.max() / scale:.3e}"
    tol = ulps * 2.0 ** -8 * np.abs(ref) + 2.0 ** -9 * scale * 1e-1 + 1e-30
    bad = err > tol
    assert bad.mean() <= 1e-3, f"{what}: {bad.mean():.3%} of entries beyond {ulps} bf16 ulps"


def oracle_spmm(x, m):
    return O.bcsr_spmm(x, m["codes"], m["scales"], m["col_idx"], m["offsets"])
