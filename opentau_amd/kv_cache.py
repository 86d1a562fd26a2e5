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
        self._ids = None        # the block ids whose summary the workspace holds
        self._workspace = None

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
        self._ids = None

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
        The same tuple object passed again (every layer and denoise step does) reuses the key-tile summary.
        ``n > 1``: candidates of best-of-N sampling, in ``(b n)`` order, share cache entry ``b``.  Inference
        only.
        """
        q_blk, k_blk, q_valid, k_valid = attention_block_ids
        scale = scaling if scaling is not None else query_states.shape[-1] ** -0.5
        kc, vc = self.layer(layer)
        ready = self._ids is attention_block_ids and self._workspace is not None
        if not ready:
            self._workspace = self._sized_workspace(query_states, kc, key_states)
        out, _ = fa.forward_raw(query_states, kc, vc, q_blk, k_blk, q_valid, k_valid, scale, key_states, value_states,
                                kvcache=True, workspace=self._workspace, summary_ready=ready, want_lse=False)
        self._ids = attention_block_ids
        return out.reshape(out.shape[0], out.shape[1], -1)

    def _sized_workspace(self, q, kc, k_new) -> torch.Tensor:
        need = fa.kvcache_workspace_bytes(q.shape[0], q.shape[1], kc.shape[1], k_new.shape[1], q.shape[2], kc.shape[2],
                                          q.shape[3], q.dtype)
        ws = self._workspace
        if ws is None or ws.numel() < need or ws.device != q.device:
            ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
        return ws
