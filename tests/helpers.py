"""Shared test plumbing: golden-fixture loading and oracle <-> product adapters."""

from __future__ import annotations

import json
import os
from types import SimpleNamespace

import numpy as np
import torch

from oracle import tq_oracle as O

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


class Golden:
    """Lazy access to tests/golden/*.npz; 16-bit floats come back as torch tensors
    of their real dtype (they are stored as raw bit patterns)."""

    def __init__(self):
        self._files = {}

    def npz(self, name):
        if name not in self._files:
            self._files[name] = np.load(os.path.join(GOLDEN_DIR, name + ".npz"))
        return self._files[name]

    def tensor(self, file, key) -> torch.Tensor:
        z = self.npz(file)
        if key in z.files:
            return torch.from_numpy(z[key].copy())
        bits = torch.from_numpy(z[key + "_bits"].copy())
        tag = str(z[key + "_dtype"])
        return bits.view(torch.bfloat16 if tag == "bf16" else torch.float16)

    def has(self, file, key) -> bool:
        z = self.npz(file)
        return key in z.files or (key + "_bits") in z.files

    def cases(self, file):
        return sorted({k.split(".")[0] for k in self.npz(file).files if "." in k})

    def json(self, name):
        with open(os.path.join(GOLDEN_DIR, name)) as f:
            return json.load(f)

    def codebook(self, d, bits):
        return self.json(f"ref_codebook_d{d}_b{bits}.json")

    def key_case_list(self):
        """(file, case) of every golden key-quantiser case."""
        return [(f, c) for f in ("key_cases", "key_cases_wide") for c in self.cases(f)]

    def key_params(self, file, case) -> O.KeyParams:
        d, bits, seed = [int(v) for v in self.npz(file)[case + ".meta"]]
        if self.has(file, case + ".S"):
            S = self.tensor(file, case + ".S")
        else:       # not stored for the widest case: S is torch.randn of seed + 1000, which is bit-stable
            S = torch.randn(d, d, generator=torch.Generator().manual_seed(seed + 1000))
        return O.KeyParams(self.tensor(file, case + ".Pi"), S,
                           self.tensor(file, case + ".centroids"), self.tensor(file, case + ".thresholds"), bits - 1)


def key_code(idx, signs, rnorms, norms, mse_bits):
    return SimpleNamespace(mse_indices=idx, qjl_signs=signs, residual_norms=rnorms, norms=norms, mse_bits=mse_bits)


def value_code(data, scales, zeros, bits):
    return SimpleNamespace(data=data, scales=scales, zeros=zeros, bits=bits)


def install_matrices(tq, prm: O.KeyParams):
    """Make a product quantiser use exactly the oracle's Pi / S / codebook (Pi
    from torch.linalg.qr is not bit-reproducible across hosts, so it travels as data)."""
    dev = tq.S.device
    mq = tq.mse_quantizer
    mq.Pi.copy_(prm.Pi.to(dev))
    mq._PiT = mq.Pi.T.contiguous()
    tq.S.copy_(prm.S.to(dev))
    tq._ST = tq.S.T.contiguous()
    mq.centroids.copy_(prm.centroids.to(dev))
    mq.decision_boundaries.copy_(prm.thresholds.to(dev))
    mq._centroids_host = prm.centroids.clone().float()
    return tq


def params_of(tq) -> O.KeyParams:
    mq = tq.mse_quantizer
    return O.KeyParams(mq.Pi.detach().cpu(), tq.S.detach().cpu(), mq.centroids.detach().cpu(),
                       mq.decision_boundaries.detach().cpu(), mq.bits)


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm() + 1e-300))


def byte_mismatch(a: torch.Tensor, b: torch.Tensor) -> int:
    return int((a.cpu() != b.cpu()).sum())


def bit_mismatch(a: torch.Tensor, b: torch.Tensor) -> int:
    x = (a.cpu().to(torch.int32) ^ b.cpu().to(torch.int32)).numpy().astype(np.uint8)
    return int(np.unpackbits(x).sum())
