"""Shared test helpers: seeded synthetic inputs of the benchmark configurations,
bf16 <-> bit-pattern conversions, and comparison utilities."""
from __future__ import annotations

import numpy as np
import torch


# name -> (M, N, K, KN, KS, KO)
CONFIGS = {
    "c0": (128, 4096, 4096, 2560, 1408, 128),
    "c1": (4096, 0, 4096, 2560, 1408, 128),
    "c2": (8, 14336, 4096, 2560, 1408, 128),
    "c3": (4096, 14336, 4096, 2560, 1408, 128),
    "c4": (2048, 4096, 14336, 8960, 4928, 448),
}


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor (any device) -> uint16 numpy bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().float().numpy()


def make_activations(m, k, seed, n_out=None, student_t=False, outlier_scale=30.0):
    g = torch.Generator().manual_seed(seed)
    if student_t:
        z = torch.randn(m, k, generator=g)
        chi = torch.randn(3, m, k, generator=g).pow(2).sum(0) / 3.0
        x = z / chi.sqrt()
    else:
        x = torch.randn(m, k, generator=g)
    if n_out is None:
        n_out = k // 32
    cols = torch.randperm(k, generator=g)[:n_out]
    x[:, cols] *= outlier_scale
    return x.to(torch.bfloat16)


def make_weights(n, k, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, k, generator=g) * std).to(torch.bfloat16)


def absmax_sort_index(x: torch.Tensor) -> torch.Tensor:
    """Channels sorted by absmax ascending (stable), int16: outliers end up in the
    last (MXFP8) segment."""
    amax = x.float().abs().amax(dim=0)
    return torch.sort(amax, stable=True).indices.to(torch.int16)


def random_index(k, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randperm(k, generator=g).to(torch.int16)


def gather_logical_scales(sf: torch.Tensor, rows: int, kseg: int) -> np.ndarray:
    from oracle import mx_oracle as mo   # imported where it is used: bench.py takes its inputs from this module
    return mo.sf_gather(sf.detach().cpu().numpy(), rows, kseg)


def assert_quant_equal(got, want, rows, splits, what=""):
    """got: 6 device tensors; want: dict from the oracle (packed codes + laid-out
    scale buffers).  Codes bit-exact; scales compared at the logical entries only
    (rows past the end of the matrix are never written)."""
    from oracle import mx_oracle as mo
    names = ("qn", "qs", "qo")
    for t, name in zip(got[:3], names):
        np.testing.assert_array_equal(t.cpu().numpy(), want[name], err_msg=f"{what} {name}")
    for t, name, kseg in zip(got[3:], ("sfn", "sfs", "sfo"), splits):
        a = gather_logical_scales(t, rows, kseg)
        b = mo.sf_gather(want[name], rows, kseg)
        np.testing.assert_array_equal(a, b, err_msg=f"{what} {name}")


def bf16_ulp(ref: np.ndarray) -> np.ndarray:
    """Spacing of bf16 at |ref| (ref float32)."""
    a = np.abs(ref).astype(np.float32)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -126)))
    return np.ldexp(1.0, (e - 7).astype(np.int32)).astype(np.float32)
