"""Loader for the fixtures in tests/golden/ (format described in tests/golden/make_golden.py)."""

from __future__ import annotations

import pathlib

import numpy as np
import torch

GOLDEN_DIR = pathlib.Path(__file__).resolve().parent / "golden"
NAMES = sorted(p.stem for p in GOLDEN_DIR.glob("*.npz"))


def load(name: str) -> dict:
    with np.load(GOLDEN_DIR / f"{name}.npz", allow_pickle=False) as z:
        dtype = getattr(torch, str(z["dtype"]))
        out = {"dtype": dtype, "scale": float(z["scale"])}
        for key in ("q", "k", "v", "d_o"):
            out[key] = torch.from_numpy(z[key].view(np.int16).copy()).view(dtype)
        for key in ("o", "lse", "delta", "dq", "dk", "dv"):
            out[key] = torch.from_numpy(z[key].copy())
    return out
