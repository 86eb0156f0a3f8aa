"""Writes the golden fixtures of this directory.

The reference ships no stored vectors for this path (its tests draw inputs from the GPU RNG and
compare with naive attention on the fly), so these fixtures come from this repository's own fp64
closed-form oracle, itself pinned in tests/test_oracle.py.  Each .npz holds the half-precision
inputs as raw 16-bit patterns plus the fp64-computed expectations stored as fp32:
q, k, v, d_o (uint16), dtype ("float16" | "bfloat16"), scale, o, lse, delta, dq, dk, dv.

    python tests/golden/make_golden.py
"""

from __future__ import annotations

import pathlib
import sys

import numpy as np
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
from oracle import naive_attention as oracle  # noqa: E402

HERE = pathlib.Path(__file__).resolve().parent

CASES = {
    # name: (batch, heads, seqlen_q, seqlen_k, headdim, dtype, qk_std, scale)
    "ragged_fp16_n75_d64": (1, 2, 75, 75, 64, torch.float16, 1.0, None),
    "peaky_fp16_n150_d64": (1, 2, 150, 150, 64, torch.float16, 3.0, None),
    "bf16_nq96_nk80_d48": (1, 2, 96, 80, 48, torch.bfloat16, 1.0, 0.2),
    "bf16_n200_d128": (1, 1, 200, 200, 128, torch.bfloat16, 1.0, None),
}


def main() -> None:
    for name, (b, h, nq, nk, d, dtype, std, scale) in CASES.items():
        gen = torch.Generator().manual_seed(42)
        q = (torch.randn(b, h, nq, d, generator=gen) * std).to(dtype)
        k = (torch.randn(b, h, nk, d, generator=gen) * std).to(dtype)
        v = torch.randn(b, h, nk, d, generator=gen).to(dtype)
        d_o = torch.randn(b, h, nq, d, generator=gen).to(dtype)
        o, dq, dk, dv = oracle.closed_form_backward(q, k, v, d_o, scale, torch.float64)
        lse = oracle.naive_lse(q, k, scale, torch.float64)
        delta = oracle.naive_delta(o, d_o, torch.float64)
        bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)  # noqa: E731
        f32 = lambda t: t.to(torch.float32).numpy()  # noqa: E731
        np.savez_compressed(
            HERE / f"{name}.npz",
            q=bits(q), k=bits(k), v=bits(v), d_o=bits(d_o),
            dtype=np.array(str(dtype).replace("torch.", "")),
            scale=np.array(scale if scale is not None else d ** -0.5, dtype=np.float64),
            o=f32(o), lse=f32(lse), delta=f32(delta), dq=f32(dq), dk=f32(dk), dv=f32(dv),
        )
        print("wrote", name)


if __name__ == "__main__":
    main()
