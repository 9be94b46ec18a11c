"""Shared helpers for the parity tests: torch <-> oracle array conversion and synthetic inputs."""
import numpy as np
import torch


def to_oracle(t):
    """torch tensor (bf16/f32/u8, any device) -> numpy array in the oracle's convention (bf16 as uint16 bits)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def from_oracle_bf16(a):
    return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)


def sign_int(signs):
    """+-1 vector -> python int bit mask (bit j set = column j negated)."""
    m = 0
    for j, s in enumerate(signs.tolist()):
        if s < 0:
            m |= 1 << j
    return m


def make_input(rows, cols, dtype, seed, outlier_frac=1e-3, scale=1.0, zero_rows=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) * scale
    if outlier_frac:
        m = torch.rand(rows, cols, generator=g) < outlier_frac
        sgn = torch.where(torch.rand(rows, cols, generator=g) < 0.5, -1.0, 1.0)
        x = torch.where(m, 1e3 * sgn * scale, x)
    if zero_rows:
        x[:zero_rows] = 0
    return x.to(dtype)
