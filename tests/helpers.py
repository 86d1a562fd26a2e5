"""Shared builders for the attention tests (mask patterns follow the reference's
``tests/policies/test_flash_attn_cuda.py:42-88``)."""

from __future__ import annotations

import torch

from opentau_amd.flash_attn_hip import make_att_block_ids

PATTERNS = ["causal", "prefixlm", "multiblock", "bidir"]


def att_masks(pattern: str, b: int, n: int) -> torch.Tensor:
    att = torch.zeros(b, n, dtype=torch.int32)
    if pattern == "causal":
        att[:] = 1
    elif pattern == "prefixlm":
        att[:, n // 2 :] = 1
    elif pattern == "multiblock":
        att[:, :: max(1, n // 5)] = 1
    elif pattern == "bidir":
        pass
    else:
        raise ValueError(pattern)
    return att


def make_blocks(b, n, pattern, cross=0, pad_tail=0, pad_mid=None):
    """Block ids as the reference's ``_make_blocks``; ``pad_mid=(lo,hi)`` adds a hole on sample 1."""
    pad = torch.ones(b, n, dtype=torch.bool)
    if pad_tail:
        pad[0, -pad_tail:] = False
    if pad_mid is not None and b > 1:
        pad[1, pad_mid[0] : pad_mid[1]] = False
    att = att_masks(pattern, b, n)
    if cross:
        cross_pad = torch.ones(b, cross, dtype=torch.bool)
        cross_pad[0, -1:] = False
        return make_att_block_ids(pad, att, cross, cross_pad)
    return make_att_block_ids(pad, att)


def randn(shape, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a, b):
    return float((a.double() - b.double()).abs().max())


def assert_close_bf16(got, ref, what, rel=1e-2, mabs=2e-2):
    """The acceptance bar for bf16 outputs and gradients: rel-L2 <= 1e-2 and max-abs <= 2e-2."""
    r, m = rel_l2(got, ref), max_abs(got, ref)
    assert r <= rel and m <= mabs, f"{what}: rel-L2 {r:.3e} (<= {rel}), max-abs {m:.3e} (<= {mabs})"
    return r, m


def assert_close_f32(got, ref, what, rel=1e-5):
    """The acceptance bar for the fp32 path: rel-L2 <= 1e-5."""
    r = rel_l2(got, ref)
    assert r <= rel, f"{what}: rel-L2 {r:.3e} (<= {rel})"
    return r
