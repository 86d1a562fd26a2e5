"""Model-facing attention calls of the policies, on the HIP kernels.

These are the call sites a policy's ``_run_layer`` reaches
(``src/opentau/policies/pi05/paligemma_with_expert.py:758-768``,
``src/opentau/policies/pi06/gemma3_with_expert.py:893-903``,
``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:230``), with the same
argument order and the same ``(B, Sq, H*D)`` result, but fed by block ids
instead of a dense ``(B, Sq, Sk)`` mask.  The functions take ``self`` first so
they can be bound onto the reference's model classes, and ignore it.
"""

from __future__ import annotations

import torch

from .flash_attn_hip import (
    BlockIds,
    flash_attn_blockmask,
    flash_attn_blockmask_kvcache,
    make_att_block_ids,
)

ATTENTION_IMPLEMENTATION = "flash_hip"


def _held(attention_block_ids) -> BlockIds | None:
    return attention_block_ids if isinstance(attention_block_ids, BlockIds) else None


def flash_hip_active(attention_implementation: str) -> bool:
    """True when this backend is selected (no fallback when it is)."""
    return attention_implementation == ATTENTION_IMPLEMENTATION


def build_attention_inputs(
    use_flash: bool,
    pad_masks: torch.Tensor,
    att_masks: torch.Tensor,
    n_cross_att_tokens: int | None = None,
    cross_att_pad_masks: torch.Tensor | None = None,
):
    """``(attention_mask, attention_block_ids)`` for the active backend.

    Counterpart of ``build_attention_inputs`` in
    ``src/opentau/policies/pi07_paligemma/low_level/modeling_pi07_low_level.py:257-275``.
    With ``use_flash`` the dense mask is never built and ``attention_mask`` is
    ``None``.  The block ids come as a :class:`BlockIds`, which unpacks like the reference's tuple and
    lets the calls below prepare the kernels' view of the mask once for all layers.  Without it this backend has nothing to offer: the dense-mask
    backends belong to the caller, so it raises.
    """
    if not use_flash:
        raise RuntimeError(
            "build_attention_inputs(use_flash=False): the dense-mask backends (eager, sdpa) are the "
            "caller's; this package only serves the block-id backend"
        )
    return None, BlockIds(*make_att_block_ids(pad_masks, att_masks, n_cross_att_tokens, cross_att_pad_masks))


def flash_attention_forward(
    self,  # noqa: ARG001
    attention_block_ids: tuple[torch.Tensor, ...],
    batch_size: int,
    head_dim: int,
    query_states: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    scaling: float | None = None,
) -> torch.Tensor:
    """``q (B,Sq,H,D), k/v (B,Sk,Hkv,D) -> (B, Sq, H*D)``.

    Same contract as ``flash_attention_forward`` in
    ``src/opentau/policies/pi05/paligemma_with_expert.py:844-880``; the optional
    ``scaling`` is the keyword of the Gemma-3 variant
    (``src/opentau/policies/pi06/gemma3_with_expert.py:525-575``) and defaults to
    ``head_dim ** -0.5``.
    """
    q_blk, k_blk, q_valid, k_valid = attention_block_ids
    scale = scaling if scaling is not None else head_dim**-0.5
    out = flash_attn_blockmask(query_states, key_states, value_states, q_blk, k_blk, q_valid, k_valid, scale,
                               block_ids=_held(attention_block_ids))
    return out.reshape(batch_size, out.shape[1], -1)


def flash_attention_forward_kvcache(
    self,  # noqa: ARG001
    attention_block_ids: tuple[torch.Tensor, ...],
    batch_size: int,
    head_dim: int,
    query_states: torch.Tensor,
    cache_key_states: torch.Tensor,
    cache_value_states: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    scaling: float | None = None,
) -> torch.Tensor:
    """The ``use_cache`` branch of ``_run_layer`` without the ``torch.cat``.

    Equivalent to concatenating ``past_key_values[layer]`` with this step's K/V
    (``src/opentau/policies/pi05/paligemma_with_expert.py:747-748``) and calling
    :func:`flash_attention_forward`; ``attention_block_ids`` cover the
    concatenation, as ``make_att_block_ids(pad, att, n_cross, cross_pad)`` builds
    them.
    """
    q_blk, k_blk, q_valid, k_valid = attention_block_ids
    scale = scaling if scaling is not None else head_dim**-0.5
    out = flash_attn_blockmask_kvcache(
        query_states, cache_key_states, cache_value_states, key_states, value_states, q_blk, k_blk, q_valid,
        k_valid, scale, block_ids=_held(attention_block_ids),
    )
    return out.reshape(batch_size, out.shape[1], -1)


def attend_bhsd(
    self,  # noqa: ARG001
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    attention_block_ids: tuple[torch.Tensor, ...],
    scaling: float | None = None,
) -> torch.Tensor:
    """Head-major layout: ``q (B,Hq,Sq,hd)``, ``k,v (B,Hkv,Sk,hd)`` -> ``(B,Sq,Hq*hd)``.

    Counterpart of ``Qwen3ExpertAttention._attend``
    (``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:188-206``).  The
    transposes are views; the kernels read the head-major strides directly.
    """
    q_blk, k_blk, q_valid, k_valid = attention_block_ids
    scale = scaling if scaling is not None else q.shape[-1] ** -0.5
    out = flash_attn_blockmask(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), q_blk, k_blk, q_valid, k_valid, scale,
        block_ids=_held(attention_block_ids),
    )
    return out.reshape(out.shape[0], out.shape[1], -1)


def attend_bhsd_kvcache(
    self,  # noqa: ARG001
    q: torch.Tensor,
    cached_kv: tuple[torch.Tensor, torch.Tensor],
    k: torch.Tensor,
    v: torch.Tensor,
    attention_block_ids: tuple[torch.Tensor, ...],
    scaling: float | None = None,
) -> torch.Tensor:
    """``Qwen3ExpertAttention.forward``'s cat + ``_attend``
    (``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:226-230``) in one call."""
    q_blk, k_blk, q_valid, k_valid = attention_block_ids
    scale = scaling if scaling is not None else q.shape[-1] ** -0.5
    ck, cv = cached_kv
    out = flash_attn_blockmask_kvcache(
        q.transpose(1, 2), ck.transpose(1, 2), cv.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
        q_blk, k_blk, q_valid, k_valid, scale, block_ids=_held(attention_block_ids),
    )
    return out.reshape(out.shape[0], out.shape[1], -1)
