"""Writes the golden fixtures of this folder (run from the repository root:
``python tests/golden/make_fixtures.py``).

The reference ships no golden vectors for its attention path, so these are made here, on the
CPU, by the float64 brute force in C (``oracle/bcattn_ref.c``: a double loop over (query, key)
pairs and the closed-form backward) from seeded inputs that the tests regenerate.  One file per
mask pattern of the reference's kernel tests (``tests/policies/test_flash_attn_cuda.py:42-88``)
plus the cross-attention layout of its KV-cache tests (``:146-162``), each holding the expected
output, log-sum-exp and gradients in float32.  They pin the eager oracle (CPU test) and the HIP
kernels in fp32, bf16 and fp16 (GPU tests) to answers that no test run computes.

The ``rope_*`` files do the same for the rotary embedding: float64, element by element, through
complex multiplication (``oracle/rope.py: rope_closed_form``), for plain positions and for three
interleaved MRoPE axes.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from helpers import PATTERNS, make_blocks, randn  # noqa: E402
from oracle import bruteforce  # noqa: E402
from oracle import rope as oracle_rope  # noqa: E402

# name -> (pattern, batch, queries, cross keys, heads, kv heads, head_dim)
CASES = {p: (p, 1, 24, 0, 2, 1, 64) for p in PATTERNS}
CASES["cross"] = ("prefixlm", 1, 17, 12, 4, 2, 64)


def case_inputs(name: str, dtype=torch.float32):
    """The seeded inputs of a fixture: q, k, v, d_out (cast to ``dtype``), ids, scale."""
    pattern, b, sq, cross, h, hkv, d = CASES[name]
    seed = 1000 + sorted(CASES).index(name) * 10
    ids = make_blocks(b, sq, pattern, cross=cross, pad_tail=0 if cross else 3)
    q = randn((b, sq, h, d), dtype, seed + 1)
    k = randn((b, cross + sq, hkv, d), dtype, seed + 2)
    v = randn((b, cross + sq, hkv, d), dtype, seed + 3)
    d_out = randn((b, sq, h, d), dtype, seed + 4) * ids[2][:, :, None, None].to(dtype)
    return q, k, v, d_out, ids, d**-0.5


# name -> (batch, tokens, heads, head_dim, MRoPE axes (0: plain positions), max wavelength)
ROPE_CASES = {"rope_1d": (2, 9, 3, 32, 0, 10_000), "rope_mrope": (1, 7, 2, 48, 3, 1_000_000)}


def rope_inputs(name: str, dtype=torch.float32):
    """The seeded inputs of a rotary fixture: x (cast to ``dtype``), positions, max wavelength."""
    b, length, h, d, axes, w = ROPE_CASES[name]
    seed = 2000 + sorted(ROPE_CASES).index(name) * 10
    x = randn((b, length, h, d), dtype, seed + 1)
    gen = torch.Generator().manual_seed(seed + 2)
    positions = torch.randint(0, 50, (axes, b, length) if axes else (b, length), generator=gen)
    return x, positions, w


def main() -> None:
    out_dir = Path(__file__).resolve().parent
    for name in ROPE_CASES:
        x, positions, w = rope_inputs(name)
        out = oracle_rope.rope_closed_form(x, positions, w)
        np.savez_compressed(out_dir / f"{name}.npz", out=out.to(torch.float32).numpy())
        print(name, tuple(out.shape), f"{(out_dir / f'{name}.npz').stat().st_size} bytes")
    for name in CASES:
        q, k, v, d_out, ids, scale = case_inputs(name)
        out, lse = bruteforce.fwd(q, k, v, *ids, scale)
        dq, dk, dv = bruteforce.bwd(q, k, v, d_out, *ids, scale)
        np.savez_compressed(out_dir / f"{name}.npz", **{
            key: t.to(torch.float32).numpy() for key, t in dict(out=out, lse=lse, dq=dq, dk=dk, dv=dv).items()
        })
        print(name, tuple(out.shape), f"{(out_dir / f'{name}.npz').stat().st_size} bytes")


if __name__ == "__main__":
    main()
