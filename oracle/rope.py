"""CPU oracle for the rotary position embedding (and the per-head RMS norm that can precede it).
TEST INFRASTRUCTURE ONLY: nothing in the product package may import this module; ``tests/`` and
the ``cpu_baseline`` leg of ``bench.py`` use it as the checker.

``apply_rope`` restates ``apply_rope`` of the reference
(``src/opentau/policies/pi05/paligemma_with_expert.py:52-107``; pi0, pi06 and pi07 carry the same
function) in plain PyTorch, so it runs on CPU or on a GPU tensor alike.  ``gemma3_rms_norm``
restates ``Gemma3RMSNorm.forward`` of the third-party dependency ``transformers`` (pinned
``>=4.57,<4.58`` by the reference's ``pyproject.toml:79``; the reference calls it as
``layer.self_attn.q_norm`` / ``k_norm`` at ``src/opentau/policies/pi06/gemma3_with_expert.py:851-861``).

What pins them (``tests/test_oracle_rope.py``):

* ``apply_rope``       the reference's own tests (``tests/policies/test_pi06.py:159-180``: shape and
                       dtype kept, different wavelengths differ, position 0 is the identity); the
                       closed form ``(x1 + i x2) * exp(i * pos / w**(2d/D))`` evaluated in float64 with
                       Python complex numbers, per element (``rope_closed_form``), which fixes the
                       pairing d <-> d + D/2, the sign of the rotation and the frequency of every band;
                       |x1|^2 + |x2|^2 kept; rotations compose by adding positions; the docstring's
                       claim that equal MRoPE axes reproduce 1-D RoPE bit for bit (``:62-64``); distinct
                       axes against the closed form (band d follows axis d % A).
* ``gemma3_rms_norm``  float64 closed form; weight 0 on unit-RMS rows is the identity; a scaled row
                       gives the same result (scale invariance up to eps).
* ``apply_rotary_pos_emb``  (restates the function of that name in ``transformers``'
                       ``models/qwen3_vl/modeling_qwen3_vl.py``, which
                       ``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:70`` imports and ``:224`` calls)
                       the library routine itself where ``transformers`` is importable, bit for bit in
                       bf16 and fp32; in fp32 with cos / sin of the same angles it equals ``apply_rope``
                       and the complex closed form; and a bf16 case built so that rounding each
                       product separately gives another answer than rounding the sum once.
* ``expert_rms_norm``  (``ExpertRMSNorm.forward``, ``cosmos3/qwen3vl_with_expert.py:85-102``) float64
                       closed form; weight 1 on unit-RMS rows is the identity; the two roundings
                       (normalised value, then the product with the weight) shown on a bf16 case.

No function here is "parity unpinned".
"""

from __future__ import annotations

import cmath

import torch


def apply_rope(x: torch.Tensor, positions: torch.Tensor, max_wavelength: float = 10_000) -> torch.Tensor:
    """``x (B, L, H, D)``; ``positions (B, L)`` or ``(A, B, L)``.  fp32 arithmetic, result in ``x.dtype``
    (reference ``paligemma_with_expert.py:79-107``)."""
    d = x.shape[-1]
    half = d // 2
    xf = x.to(torch.float32)
    band = torch.arange(half, dtype=torch.float32, device=x.device)
    timescale = max_wavelength ** ((2.0 / d) * band)  # :84-85
    pos = positions.to(torch.float32)
    if positions.ndim == 3:  # interleaved MRoPE: band i follows axis i % A (:90-97)
        axis_of_band = torch.arange(half, device=x.device) % positions.shape[0]
        pos = pos[axis_of_band].permute(1, 2, 0)  # (B, L, half)
    else:
        pos = pos.unsqueeze(-1)
    angle = (pos / timescale).unsqueeze(-2)  # one angle per (token, band), shared by the heads (:99)
    s, c = torch.sin(angle), torch.cos(angle)
    lo, hi = xf[..., :half], xf[..., half:]
    out = torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)  # :104-105
    return out.to(x.dtype)


def gemma3_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * (1 + weight)`` in fp32 over the last axis, then back to ``x.dtype``
    (``transformers/models/gemma3/modeling_gemma3.py``, ``Gemma3RMSNorm.forward``)."""
    xf = x.to(torch.float32)
    normed = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (normed * (1.0 + weight.to(torch.float32))).to(x.dtype)


def rope_closed_form(x, positions, max_wavelength: float = 10_000):
    """Float64, element by element, through complex multiplication.  ``x`` nested lists / tensor
    ``(B, L, H, D)``, ``positions (B, L)`` or ``(A, B, L)``.  Small inputs only."""
    x = torch.as_tensor(x, dtype=torch.float64)
    positions = torch.as_tensor(positions)
    b_n, l_n, h_n, d = x.shape
    half = d // 2
    out = torch.empty_like(x)
    for b in range(b_n):
        for l in range(l_n):  # noqa: E741
            for i in range(half):
                if positions.ndim == 3:
                    p = float(positions[i % positions.shape[0], b, l])
                else:
                    p = float(positions[b, l])
                turn = cmath.exp(1j * p / float(max_wavelength) ** (2.0 * i / d))
                for h in range(h_n):
                    z = complex(float(x[b, l, h, i]), float(x[b, l, h, i + half])) * turn
                    out[b, l, h, i], out[b, l, h, i + half] = z.real, z.imag
    return out


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim: int = 1):
    """``x * cos + rotate_half(x) * sin`` for q and k, in the tensors' own dtype (each elementwise op rounds);
    ``cos`` / ``sin`` ``(B, S, D)`` are broadcast over the head axis at ``unsqueeze_dim``."""
    c, s = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return q * c + rotate_half(q) * s, k * c + rotate_half(k) * s


def expert_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``weight * (x * rsqrt(mean(x^2) + eps)).to(x.dtype)``, the statistics in fp32
    (``cosmos3/qwen3vl_with_expert.py:97-102``)."""
    xf = x.to(torch.float32)
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (weight * xf.to(x.dtype)).to(x.dtype)


def rope_tables(positions: torch.Tensor, head_dim: int, max_wavelength: float = 10_000, dtype=torch.float32):
    """``(cos, sin)`` ``(B, S, D)`` of plain positions ``(B, S)`` with both halves alike, the layout the
    rotary module of a Hugging Face text model returns (``emb = cat(freqs, freqs)``)."""
    half = head_dim // 2
    timescale = max_wavelength ** ((2.0 / head_dim) * torch.arange(half, dtype=torch.float32, device=positions.device))
    freqs = positions.to(torch.float32).unsqueeze(-1) / timescale
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def norm_rope_backward(x, weight, grad_out, *, kind, positions=None, max_wavelength: float = 10_000, cos=None,
                       sin=None, eps: float = 1e-6):
    """``(dx, dweight)`` of the per-head norm followed by the rotation, by autograd through the functions
    above.  ``kind`` ``"gemma3"``: ``x (B, L, H, D)``, ``apply_rope(gemma3_rms_norm(x))`` with ``positions``
    (``pi06/gemma3_with_expert.py:851-861``); ``"qwen3"``: ``x (B, H, S, D)``, the expert's norm then
    ``apply_rotary_pos_emb`` with ``cos`` / ``sin`` (``cosmos3/qwen3vl_with_expert.py:217-224``)."""
    x = x.detach().clone().requires_grad_(True)
    weight = weight.detach().clone().requires_grad_(True)
    if kind == "gemma3":
        out = apply_rope(gemma3_rms_norm(x, weight, eps), positions, max_wavelength)
    else:
        out = apply_rotary_pos_emb(expert_rms_norm(x, weight, eps), x[:, :0], cos, sin)[0]
    out.backward(grad_out)
    return x.grad, weight.grad
