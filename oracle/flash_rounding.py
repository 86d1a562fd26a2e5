"""Float64 model of where a flash-attention kernel rounds. TEST INFRASTRUCTURE ONLY.

The eager oracle (``oracle/eager.py``) keeps the whole score matrix and rounds the probabilities once.
A flash kernel, the reference's as well as this build's, differs in three places
(``src/opentau/policies/flash_attn_cuda/_csrc/flash_blockmask.cu``):

* ``delta = rowsum(O * dO)`` is taken from the *stored* output, i.e. O rounded to the 16-bit element
  type (``:249-269``), not from the fp32 probabilities;
* P and dS enter the second product of each pair as 16-bit MMA operands (``:821`` "P = exp(scale*S - L);
  dS = P*(dP - delta)" into the half-precision tiles);
* everything else (dot products of exact 16-bit values) is summed in fp32, modelled here as exact.

``flash_grads_rounded`` computes O, dQ, dK, dV in float64 with exactly those roundings switched on or
off.  With all of them off it is the textbook closed form and is pinned as such: against ``torch.autograd``
through the eager oracle in float64 and against the float64 brute force (``tests/test_oracle.py``).  It is
used to tell rounding from defects where a gradient is a small difference of large terms (one query
row, peaked softmax), and only by tests.
"""

from __future__ import annotations

import torch

from .eager import dense_mask_from_block_ids


def _rounded(x: torch.Tensor, dtype) -> torch.Tensor:
    return x if dtype is None else x.to(dtype).double()


def flash_grads_rounded(q, k, v, d_out, q_blk, k_blk, q_valid, k_valid, scale, *, round_o=True, round_p=True,
                        round_ds=True, o_stored=None, lse_stored=None):
    """``(O, dQ, dK, dV)`` in float64; rounding points use the dtype of ``q`` (none for float64 inputs).

    ``o_stored (B,Sq,H,D)`` / ``lse_stored (B,H,Sq)``: what a forward pass left in memory.  A flash
    backward is a function of those (``delta`` from the stored O, ``P = exp(scale*S - LSE)`` from the
    stored LSE); passing them models the backward of that very forward, so that the comparison does
    not depend on how the forward's rounding fell."""
    dtype = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else None
    mask = dense_mask_from_block_ids(q_blk, k_blk, q_valid, k_valid)  # (B,Sq,Sk)
    b, sq, h, d = q.shape
    hkv = k.shape[2]
    grp = h // hkv
    qf, gf = q.double(), d_out.double() * q_valid[:, :, None, None]
    kf = k.double().repeat_interleave(grp, 2)
    vf = v.double().repeat_interleave(grp, 2)
    s = torch.einsum("bihd,bjhd->bhij", qf, kf) * scale
    s = s.masked_fill(~mask[:, None], float("-inf"))
    row_has_key = mask.any(-1)[:, None, :, None]
    lse = torch.logsumexp(torch.where(row_has_key, s, torch.zeros_like(s)), -1, keepdim=True)
    if lse_stored is not None:
        lse = lse_stored.double()[..., None]
    p = torch.where(row_has_key & mask[:, None], torch.exp(s - lse), torch.zeros_like(s))
    p16 = _rounded(p, dtype if round_p else None)
    o = torch.einsum("bhij,bjhd->bihd", p16, vf)
    o_for_delta = _rounded(o, dtype if round_o else None) if o_stored is None else o_stored.double()
    delta = (o_for_delta * gf).sum(-1).permute(0, 2, 1)[..., None]  # (B,H,Sq,1)
    dp = torch.einsum("bihd,bjhd->bhij", gf, vf)
    ds16 = _rounded(p * (dp - delta), dtype if round_ds else None)
    dq = scale * torch.einsum("bhij,bjhd->bihd", ds16, kf)
    dk = scale * torch.einsum("bhij,bihd->bjhd", ds16, qf).reshape(b, -1, hkv, grp, d).sum(3)
    dv = torch.einsum("bhij,bihd->bjhd", p16, gf).reshape(b, -1, hkv, grp, d).sum(3)
    return o, dq, dk, dv
