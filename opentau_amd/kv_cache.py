"""Preallocated prefix K/V cache of all layers, with the attention workspace shared across them.

The reference keeps ``past_key_values[layer] = {"key_states": ..., "value_states": ...}``, filled
by slicing the layer's K/V after the prefix pass
(``src/opentau/policies/pi05/paligemma_with_expert.py:749-756``), concatenates it with every
denoise step's K/V (``:747-748``; its own TODO ``:743-746`` asks for a static cache instead) and, for
best-of-N sampling, repeats it N times (``src/opentau/policies/candidates.py:114-127``).  Here the
cache is one allocation made up front; the prefix pass writes each layer's rows in place (the rotary
kernel can store the keys straight into them), a denoise step attends ``[cache ; own K/V]`` as two
segments without a copy, N candidates read one cache entry, and the key-tile summary of the mask,
which is the same for every layer and step, is computed once.
"""

from __future__ import annotations

import torch

from . import flash_attn_hip as fa
from .rope import rope_raw


class StaticKVCache:
    """``k``, ``v``: ``(layers, B, max_len, Hkv, D)``; ``length`` valid rows (the reference's
    ``n_cross_att_tokens``)."""

    def __init__(self, n_layers: int, batch: int, max_len: int, n_kv_heads: int, head_dim: int,
                 dtype: torch.dtype = torch.bfloat16, device: torch.device | str = "cuda"):
        shape = (n_layers, batch, max_len, n_kv_heads, head_dim)
        self.k = torch.empty(shape, dtype=dtype, device=device)
        self.v = torch.empty(shape, dtype=dtype, device=device)
        self.length = 0
        self._held = None  # the BlockIds (ids + workspace with their summary) of the mask in use

    @property
    def n_layers(self) -> int:
        return self.k.shape[0]

    def fill(self, layer: int, keys: torch.Tensor, values: torch.Tensor, *, positions: torch.Tensor | None = None,
             max_wavelength: float = 10_000, k_norm_weight: torch.Tensor | None = None,
             norm_eps: float = 1e-6) -> tuple[torch.Tensor, torch.Tensor]:
        """Store the first rows of a layer (the ``fill_kv_cache`` branch, ``paligemma_with_expert.py:749-756``).

        With ``positions`` the keys are still un-rotated: the rotary kernel (optionally behind the
        Gemma-3 key norm) writes them rotated into the cache rows, which replaces the layer's
        ``apply_rope(key_states, ...)``.  Returns the cache rows ``(k, v)``, which the prefix pass can
        hand to its own attention call.
        """
        n = keys.shape[1]
        if n > self.k.shape[2] or keys.shape[0] != self.k.shape[1]:
            raise RuntimeError(f"keys {tuple(keys.shape)} do not fit the cache {tuple(self.k.shape[1:])}")
        k_rows, v_rows = self.k[layer, :, :n], self.v[layer, :, :n]
        if positions is None:
            k_rows.copy_(keys)
        else:
            rope_raw(None, keys, positions, max_wavelength, k_out=k_rows, k_norm_weight=k_norm_weight,
                     norm_eps=norm_eps)
        v_rows.copy_(values)
        self.length = n
        return k_rows, v_rows

    def reset(self) -> None:
        """Forget the rows and the mask summary (a new observation; or block ids that were changed in place)."""
        self.length = 0
        self._held = None

    def layer(self, layer: int) -> tuple[torch.Tensor, torch.Tensor]:
        """The valid rows of a layer, ``(B, length, Hkv, D)`` views."""
        return self.k[layer, :, : self.length], self.v[layer, :, : self.length]

    def as_past_key_values(self) -> dict[int, dict[str, torch.Tensor]]:
        """The reference's structure (a dict keyed by layer index), as views of the cache."""
        return {i: dict(zip(("key_states", "value_states"), self.layer(i))) for i in range(self.n_layers)}

    def attend(self, layer: int, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
               attention_block_ids: tuple[torch.Tensor, ...], scaling: float | None = None) -> torch.Tensor:
        """The ``use_cache`` branch of ``_run_layer`` (``paligemma_with_expert.py:742-768``) for one layer:
        ``q (B*n, Sq, H, D)`` over ``[cache[layer] ; k, v (B*n, Sq, Hkv, D)]`` -> ``(B*n, Sq, H*D)``.

        ``attention_block_ids`` cover the concatenation (``make_att_block_ids(pad, att, n_cross, cross_pad)``).
        Every layer and denoise step passes the same ids: their tile summary is made on the first call
        and reused for as long as the id tensors stay what they were (same storage, shape and version
        counter: an in-place edit is seen, and the summary is made again).  A :class:`BlockIds`
        is used as it is.  ``n > 1``: candidates of best-of-N sampling, in ``(b n)`` order, share cache
        entry ``b``.  Inference only.
        """
        held = self._hold(attention_block_ids)
        scale = scaling if scaling is not None else query_states.shape[-1] ** -0.5
        kc, vc = self.layer(layer)
        out, _ = fa.forward_raw(query_states, kc, vc, *held, scale, key_states, value_states, kvcache=True,
                                want_lse=False, block_ids=held)
        return out.reshape(out.shape[0], out.shape[1], -1)

    def _hold(self, ids) -> fa.BlockIds:
        if isinstance(ids, fa.BlockIds):
            return ids
        held = self._held
        # the caller's own tensors, unchanged since last time (same objects, same version counters),
        # mean the same mask: the holder made from them then still stands
        source = tuple((t, t._version) for t in ids)
        if (held is None or len(source) != len(held._source)
                or any(a is not b or va != vb for (a, va), (b, vb) in zip(source, held._source))):
            held = fa.BlockIds(*ids)
            held._source = source
            self._held = held
        return held
