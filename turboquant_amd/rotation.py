"""Rotation and sketch matrices of the key quantiser.

Mirrors turboquant/rotation.py of the reference (rotation.py:17-66): the same
four functions with the same arguments.  Both matrices are drawn once per layer
on the host from a seeded CPU generator, exactly as the reference draws them,
and then live in GPU memory for the kernels.
"""

from __future__ import annotations

import torch


def _seeded_gaussian(d: int, seed: int) -> torch.Tensor:
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    return torch.randn(d, d, generator=gen, dtype=torch.float32)


def generate_rotation_matrix(d: int, device, dtype: torch.dtype = torch.float32, seed: int = 42) -> torch.Tensor:
    """Haar-distributed orthogonal Pi (d x d): the Q factor of a seeded Gaussian
    with each column multiplied by the sign of the matching diagonal entry of R.
    Its determinant can be -1; orthogonality is all the quantiser needs."""
    q_factor, r_factor = torch.linalg.qr(_seeded_gaussian(d, seed))
    col_sign = torch.sign(torch.diagonal(r_factor))
    return (q_factor * col_sign[None, :]).contiguous().to(device=device, dtype=dtype)


def generate_qjl_matrix(d: int, device, dtype: torch.dtype = torch.float32, seed: int = 12345) -> torch.Tensor:
    """i.i.d. N(0,1) sketch matrix S (d x d) for the QJL stage."""
    return _seeded_gaussian(d, seed).to(device=device, dtype=dtype)


def rotate_forward(x: torch.Tensor, Pi: torch.Tensor) -> torch.Tensor:
    """y = x Pi^T, i.e. Pi applied to every vector of x."""
    return torch.matmul(x, Pi.T)


def rotate_backward(y: torch.Tensor, Pi: torch.Tensor) -> torch.Tensor:
    """x = y Pi, the inverse of rotate_forward for an orthogonal Pi."""
    return torch.matmul(y, Pi)
