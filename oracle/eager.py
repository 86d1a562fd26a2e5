"""CPU oracle for block-causal attention. TEST INFRASTRUCTURE ONLY.

This module restates, in plain PyTorch, the reference's eager masked-softmax
attention and the mask builders that feed it.  It exists so that the HIP path
can be checked against it; nothing in the product package may import it.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and only as the checker.

Each function cites the reference file it follows (paths relative to the
reference checkout).  What pins each function (so that a dropped term, a wrong
sign or a transposed operand fails a test):

* ``make_att_2d_masks``     known answers restated from the reference's own
                            tests (all-true, ``tril``, prefix-LM rows, padding,
                            cross block ``(1,2,5)``) + a brute-force double loop.
* ``make_att_block_ids``    invariant ``dense(block ids) == make_att_2d_masks``
                            over the reference's four patterns and cross case.
* ``eager_attention_*``     ``F.scaled_dot_product_attention`` (library routine)
                            at 1e-4 in fp32, as the reference's tests do; the
                            float64 brute-force C routine in ``bcattn_ref.c``;
                            special cases (one visible key => O = V[j]; equal
                            keys => O = mean of visible V; pure causal =>
                            ``is_causal=True`` SDPA).
* backward                  ``torch.autograd`` through the eager function,
                            ``gradcheck`` in float64, the closed form in
                            ``bcattn_ref.c``.
* ``attention_lse``         ``exp(scale*S - L)`` rows sum to one.

No function here is "parity unpinned".
"""

from __future__ import annotations

import torch
import torch.nn.functional as F  # noqa: N812

INT_BLK_MIN = -(2**31)
BIG_NEG = -2.3819763e38


# --------------------------------------------------------------------------- #
# masks
# --------------------------------------------------------------------------- #
def make_att_2d_masks(pad_masks, att_masks, n_cross_att_tokens=None, cross_att_pad_masks=None):
    """Dense bool mask ``(B, N, [n_cross+]N)``, True = attend.

    Follows ``src/opentau/policies/pi05/modeling_pi05.py:120-190``: query i sees
    key j iff ``cumsum(att)[j] <= cumsum(att)[i]`` and both are valid; optional
    cross columns are prepended on the key axis and gated only by padding.
    """
    if att_masks.ndim != 2:
        raise ValueError(att_masks.ndim)
    if pad_masks.ndim != 2:
        raise ValueError(pad_masks.ndim)
    cum = torch.cumsum(att_masks, dim=1)
    att2d = cum[:, None, :] <= cum[:, :, None]
    pad2d = pad_masks[:, None, :] * pad_masks[:, :, None]
    att2d = att2d & pad2d
    if n_cross_att_tokens is not None:
        assert cross_att_pad_masks is not None
        assert cross_att_pad_masks.shape == (att_masks.size(0), n_cross_att_tokens)
        cross = pad_masks[:, :, None] & cross_att_pad_masks[:, None, :]
        att2d = torch.cat((cross, att2d), dim=2)
    return att2d


def make_att_block_ids(pad_masks, att_masks, n_cross_att_tokens=None, cross_att_pad_masks=None):
    """Compact form ``(q_blk, k_blk, q_valid, k_valid)``.

    Follows ``src/opentau/policies/flash_attn_cuda/__init__.py:58-109``.
    """
    if att_masks.ndim != 2:
        raise ValueError(att_masks.ndim)
    if pad_masks.ndim != 2:
        raise ValueError(pad_masks.ndim)
    cum = torch.cumsum(att_masks.to(torch.int32), dim=1).to(torch.int32)
    q_valid = pad_masks.to(torch.bool)
    if n_cross_att_tokens is None:
        return cum, cum, q_valid, q_valid
    assert cross_att_pad_masks is not None
    assert cross_att_pad_masks.shape == (att_masks.size(0), n_cross_att_tokens)
    b = att_masks.size(0)
    cross_blk = torch.full((b, n_cross_att_tokens), INT_BLK_MIN, dtype=torch.int32)
    k_blk = torch.cat([cross_blk, cum], dim=1)
    k_valid = torch.cat([cross_att_pad_masks.to(torch.bool), q_valid], dim=1)
    return cum, k_blk, q_valid, k_valid


def dense_mask_from_block_ids(q_blk, k_blk, q_valid, k_valid):
    """``attend(i,j) = q_valid[i] & k_valid[j] & (k_blk[j] <= q_blk[i])``.

    Follows ``src/opentau/policies/flash_attn_cuda/__init__.py:27-28`` and
    ``tests/policies/test_flash_attn_cuda.py:58-59``.
    """
    return (k_blk[:, None, :] <= q_blk[:, :, None]) & q_valid[:, :, None] & k_valid[:, None, :]


# --------------------------------------------------------------------------- #
# eager attention (the acceptance oracle)
# --------------------------------------------------------------------------- #
def eager_attention_bshd(attention_mask, q, k, v, scaling=None, fill=BIG_NEG):
    """Eager attention, ``q (B,Sq,H,D)``, ``k,v (B,Sk,Hkv,D)`` -> ``(B,Sq,H*D)``.

    Follows ``src/opentau/policies/pi05/paligemma_with_expert.py:882-953`` (and
    the ``scaling`` keyword of ``pi06/gemma3_with_expert.py:525-575``) in the
    exact order of operations: expand K/V over the query-head group; Q and K to
    fp32; ``QK^T``; times the scale; masked entries replaced by ``fill``; fp32
    softmax; probabilities cast to V's dtype; ``P @ V`` in V's dtype.
    """
    b, sq, h, d = q.shape
    sk, hkv = k.shape[1], k.shape[2]
    g = h // hkv
    k = k[:, :, :, None, :].expand(b, sk, hkv, g, d).reshape(b, sk, h, d)
    v = v[:, :, :, None, :].expand(b, sk, hkv, g, d).reshape(b, sk, h, d)
    qf = q.to(torch.float32).transpose(1, 2)
    kf = k.to(torch.float32).transpose(1, 2)
    w = torch.matmul(qf, kf.transpose(2, 3))
    w = w * (scaling if scaling is not None else d**-0.5)
    w = torch.where(attention_mask[:, None, :, :], w, fill)
    probs = F.softmax(w, dim=-1).to(v.dtype)
    out = torch.matmul(probs, v.permute(0, 2, 1, 3))
    return out.permute(0, 2, 1, 3).reshape(b, -1, h * d)


def eager_attention_bhsd(attn_mask, q, k, v, scaling=None):
    """Eager attention in head-major layout: ``q (B,Hq,Sq,hd)``, ``k,v (B,Hkv,Sk,hd)``.

    Follows ``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:78-82,188-206``:
    repeat K/V per group, fp32 scores times ``hd**-0.5``, masked entries set to
    ``finfo(float32).min``, softmax cast to V's dtype, ``P @ V``; output
    ``(B, Sq, Hq*hd)``.
    """
    b, hq, sq, d = q.shape
    n_rep = hq // k.shape[1]
    k = k.repeat_interleave(n_rep, dim=1)
    v = v.repeat_interleave(n_rep, dim=1)
    scale = scaling if scaling is not None else d**-0.5
    attn = torch.matmul(q.to(torch.float32), k.to(torch.float32).transpose(2, 3)) * scale
    attn = torch.where(attn_mask[:, None], attn, torch.finfo(torch.float32).min)
    probs = F.softmax(attn, dim=-1).to(v.dtype)
    out = torch.matmul(probs, v)
    return out.permute(0, 2, 1, 3).reshape(b, sq, hq * d)


def sdpa_attention_bshd(attention_mask, q, k, v, scaling=None):
    """Library-routine statement of the same attention (no fp32 upcast).

    Follows ``src/opentau/policies/pi05/paligemma_with_expert.py:955-1036``.
    """
    b, sq, h, d = q.shape
    g = h // k.shape[2]
    kk = k.repeat_interleave(g, dim=2).transpose(1, 2)
    vv = v.repeat_interleave(g, dim=2).transpose(1, 2)
    out = F.scaled_dot_product_attention(
        q.transpose(1, 2), kk, vv, attn_mask=attention_mask[:, None], is_causal=False, dropout_p=0.0,
        scale=scaling,
    )
    return out.permute(0, 2, 1, 3).reshape(b, sq, h * d)


def reference_attention_fp32(q, k, v, q_blk, k_blk, q_valid, k_valid, scale):
    """fp32 dense attention with ``-inf`` fill and zero rows where nothing is visible.

    Follows the helper the reference's kernel tests compare against,
    ``tests/policies/test_flash_attn_cuda.py:62-76``.  Returns
    ``(out (B,Sq,H,D) fp32, row_has_key (B,Sq) bool)``.
    """
    g = q.shape[2] // k.shape[2]
    qf = q.float().permute(0, 2, 1, 3)
    kf = k.float().permute(0, 2, 1, 3).repeat_interleave(g, dim=1)
    vf = v.float().permute(0, 2, 1, 3).repeat_interleave(g, dim=1)
    scores = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    mask = dense_mask_from_block_ids(q_blk, k_blk, q_valid, k_valid)[:, None]
    scores = scores.masked_fill(~mask, float("-inf"))
    any_key = mask.any(dim=-1, keepdim=True)
    probs = torch.where(any_key, torch.softmax(scores, dim=-1), torch.zeros_like(scores))
    out = torch.matmul(probs, vf).permute(0, 2, 1, 3).contiguous()
    return out, any_key.squeeze(1).squeeze(-1)


def attention_lse(q, k, q_blk, k_blk, q_valid, k_valid, scale):
    """Natural-log sum-exp of the masked, scaled scores, fp32 ``(B,H,Sq)``.

    Rows with no visible key hold 0, the convention of
    ``src/opentau/policies/flash_attn_cuda/_csrc/flash_blockmask.cu:240-244``.
    """
    g = q.shape[2] // k.shape[2]
    qf = q.float().permute(0, 2, 1, 3)
    kf = k.float().permute(0, 2, 1, 3).repeat_interleave(g, dim=1)
    scores = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    mask = dense_mask_from_block_ids(q_blk, k_blk, q_valid, k_valid)[:, None]
    scores = scores.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    return torch.where(mask.any(dim=-1), lse, torch.zeros_like(lse))


def eager_from_block_ids(q, k, v, q_blk, k_blk, q_valid, k_valid, scale):
    """Eager oracle driven by block ids; returns ``(B,Sq,H,D)`` in V's dtype."""
    mask = dense_mask_from_block_ids(q_blk, k_blk, q_valid, k_valid)
    b, sq, h, d = q.shape
    return eager_attention_bshd(mask, q, k, v, scaling=scale).reshape(b, sq, h, d)


def eager_grads(q, k, v, d_out, q_blk, k_blk, q_valid, k_valid, scale):
    """``(out, dq, dk, dv)`` by autograd through the eager oracle.

    ``d_out`` rows of invalid queries are zeroed first, as the reference's
    gradient tests do by masking (``tests/policies/test_flash_attn_cuda.py:191-195``):
    padded query rows get a uniform softmax in the eager path and would
    otherwise leak into dK/dV.
    """
    qr = q.detach().clone().requires_grad_(True)
    kr = k.detach().clone().requires_grad_(True)
    vr = v.detach().clone().requires_grad_(True)
    out = eager_from_block_ids(qr, kr, vr, q_blk, k_blk, q_valid, k_valid, scale)
    go = d_out * q_valid[:, :, None, None].to(d_out.dtype)
    out.backward(go)
    return out.detach(), qr.grad, kr.grad, vr.grad


def rel_l2(a, b):
    a = a.double()
    b = b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))
