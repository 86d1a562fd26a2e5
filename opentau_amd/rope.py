"""Rotary position embedding of a layer's queries and keys on the HIP kernel.

``apply_rope`` has the signature and the numerics of the reference's function of
that name (``src/opentau/policies/pi05/paligemma_with_expert.py:52-107``; the same
function serves pi0, pi06 and pi07).  ``apply_rope_qk`` is the form a layer wants:
queries and keys in one launch, optionally behind Gemma-3's per-head RMS norm
(``src/opentau/policies/pi06/gemma3_with_expert.py:851-861``), optionally written
straight into other storage such as the rows of a preallocated key cache.
``apply_rotary_pos_emb`` is the rotation of cosmos3's expert
(``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:217-224``): cos / sin tables from the
backbone's rotary module, arithmetic in the tensors' own type, optionally behind the expert's
per-head RMS norm (``:85-102``).
There is no CPU path: without the library or a HIP device the calls raise.
"""

from __future__ import annotations

import ctypes

import torch

from .flash_attn_hip import _loader
from .flash_attn_hip import _check, _DTYPES, _on_device, _stream, _t4

_timescales: dict[tuple, torch.Tensor] = {}
_NORM_KINDS = {"gemma3": 0, "qwen3": 1}  # enum bcattn_norm_kind


def rope_timescale(head_dim: int, max_wavelength: float, device: torch.device) -> torch.Tensor:
    """``max_wavelength ** (2 i / head_dim)`` for the ``head_dim / 2`` bands, fp32, computed with the
    same torch ops on the same device as ``paligemma_with_expert.py:84-85`` so the kernel divides
    by the very numbers the reference does.  Cached per (head_dim, wavelength, device).  The first
    call for a key must come outside HIP-graph capture: a tensor made while a stream is capturing lives
    in the graph's memory pool and holds data only during a replay, so it must not be kept."""
    key = (head_dim, max_wavelength, str(device))
    t = _timescales.get(key)
    if t is None:
        if torch.device(device).type == "cuda" and torch.cuda.is_current_stream_capturing():
            raise RuntimeError("rope_timescale: first use of this (head_dim, wavelength, device) under graph "
                               "capture; call the rotary embedding once before capturing")
        exponents = (2.0 / head_dim) * torch.arange(head_dim // 2, dtype=torch.float32, device=device)
        t = (max_wavelength**exponents).to(torch.float32).contiguous()
        _timescales[key] = t
    return t


def _strided(t: torch.Tensor | None, vec: int, what: str) -> torch.Tensor | None:
    if t is None:
        return None
    if t.ndim != 4:
        raise RuntimeError(f"{what} must be (B, L, H, D), got {tuple(t.shape)}")
    if t.stride(-1) != 1 or t.data_ptr() % 16 or any(s % vec for s in t.stride()[:-1]):
        raise RuntimeError(f"{what}: the head_dim axis must be contiguous, the pointer 16-byte aligned and the "
                           f"other strides multiples of {vec} elements")
    return t


def _positions(positions: torch.Tensor, b: int, length: int) -> tuple[torch.Tensor, int]:
    if positions.ndim == 2:
        n_axes = 1
    elif positions.ndim == 3:
        n_axes = positions.shape[0]
    else:
        raise RuntimeError(f"positions must be (B, L) or (A, B, L), got {tuple(positions.shape)}")
    if tuple(positions.shape[-2:]) != (b, length):
        raise RuntimeError(f"positions {tuple(positions.shape)} do not match (B, L) = {(b, length)}")
    if positions.is_floating_point():
        raise RuntimeError("positions must be integers")
    # (the kernel reads int32: positions are token indices, far below 2^31)
    return positions.to(torch.int32).contiguous(), n_axes


def rope_raw(
    q: torch.Tensor | None,
    k: torch.Tensor | None,
    positions: torch.Tensor,
    max_wavelength: float = 10_000,
    *,
    q_out: torch.Tensor | None = None,
    k_out: torch.Tensor | None = None,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    norm_eps: float = 1e-6,
    norm_kind: str = "gemma3",
    inverse: bool = False,
    cos: torch.Tensor | None = None,
    sin: torch.Tensor | None = None,
):
    """One call of ``bcattn_rope``.  Returns ``(q_out, k_out)`` (``None`` where the input is ``None``).

    ``q`` / ``k`` are ``(B, L, H, D)`` views.  With ``cos`` / ``sin`` (``(B, L, D)``, cast to the tensors'
    dtype) the rotation is ``x * cos + rotate_half(x) * sin`` in that dtype and ``positions`` is ignored.
    ``norm_kind``: ``"gemma3"`` (``x * r * (1 + w)``) or ``"qwen3"`` (``w * (x * r)``).
    """
    lib = _loader.require_library()
    x = q if q is not None else k
    if x is None:
        raise RuntimeError("rope needs q or k")
    if not x.is_cuda:
        raise RuntimeError("rope needs tensors on a HIP device; there is no CPU fallback")
    if x.dtype not in _DTYPES:
        raise RuntimeError(f"rope supports float32, bfloat16 and float16, got {x.dtype}")
    code, vec = _DTYPES[x.dtype]
    q, k = _strided(q, vec, "q"), _strided(k, vec, "k")
    b, length, d = x.shape[0], x.shape[1], x.shape[3]
    if q is not None and k is not None and (k.shape[0], k.shape[1], k.shape[3], k.dtype) != (b, length, d, q.dtype):
        raise RuntimeError(f"q {tuple(q.shape)} and k {tuple(k.shape)} differ in batch, length, head_dim or dtype")
    tables = cos is not None or sin is not None
    if tables:
        if cos is None or sin is None or tuple(cos.shape) != (b, length, d) or cos.shape != sin.shape:
            raise RuntimeError(f"cos and sin must both be (B, L, D) = {(b, length, d)}")
        cos, sin = (t.to(device=x.device, dtype=x.dtype).contiguous() for t in (cos, sin))
        pos, n_axes = None, 1
    else:
        pos, n_axes = _positions(positions, b, length)
    if norm_kind not in _NORM_KINDS:
        raise RuntimeError(f"norm_kind must be one of {sorted(_NORM_KINDS)}")
    if q is not None and q_out is None:
        q_out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if k is not None and k_out is None:
        k_out = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    for t, o, what in ((q, q_out, "q_out"), (k, k_out, "k_out")):
        if t is not None and (_strided(o, vec, what).shape != t.shape or o.dtype != t.dtype or o.device != t.device):
            raise RuntimeError(f"{what} must have the shape, dtype and device of its input")
    weights = []
    for t, w, what in ((q, q_norm_weight, "q_norm_weight"), (k, k_norm_weight, "k_norm_weight")):
        if w is not None and t is not None:
            if w.shape != (d,):
                raise RuntimeError(f"{what} must be ({d},), got {tuple(w.shape)}")
            w = w.detach().to(device=t.device, dtype=torch.float32).contiguous()
        weights.append(w if t is not None else None)
    ts = None if tables else rope_timescale(d, max_wavelength, x.device)
    p = _loader.RopeParams()
    p.q, p.k, p.q_out, p.k_out = _t4(q), _t4(k), _t4(q_out if q is not None else None), _t4(k_out if k is not None else None)
    if tables:
        p.cos, p.sin = cos.data_ptr(), sin.data_ptr()
    else:
        p.positions, p.timescale = pos.data_ptr(), ts.data_ptr()
    p.norm_kind = _NORM_KINDS[norm_kind]
    p.q_norm_weight = weights[0].data_ptr() if weights[0] is not None else None
    p.k_norm_weight = weights[1].data_ptr() if weights[1] is not None else None
    p.B, p.L, p.D = b, length, d
    p.H = q.shape[2] if q is not None else 0
    p.Hkv = k.shape[2] if k is not None else 0
    p.n_axes, p.dtype, p.inverse, p.norm_eps = n_axes, code, 1 if inverse else 0, float(norm_eps)
    with _on_device(x.device):
        _check(lib.bcattn_rope(ctypes.byref(p), _stream(x.device)), lib)
    return (q_out if q is not None else None), (k_out if k is not None else None)


def rope_norm_bwd_raw(
    grad_q: torch.Tensor | None,
    grad_k: torch.Tensor | None,
    q: torch.Tensor | None,
    k: torch.Tensor | None,
    positions: torch.Tensor | None,
    max_wavelength: float = 10_000,
    *,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    norm_eps: float = 1e-6,
    norm_kind: str = "gemma3",
    cos: torch.Tensor | None = None,
    sin: torch.Tensor | None = None,
    stacked: bool = False,
):
    """One call of ``bcattn_rope_norm_bwd``: the gradient of :func:`rope_raw` with norm weights.

    ``grad_q`` / ``grad_k``: gradients of the rotated outputs, ``q`` / ``k``: the forward's inputs, all
    ``(B, L, H, D)`` views.  Returns ``(dq, dk, dw_q, dw_k)``; the weight gradients are fp32 ``(D,)``
    (``None`` where there is no weight), the sum of the kernel's per-workgroup partial sums; with ``stacked``
    they come as one ``(2, D)`` tensor instead (a row of zeros where there is no weight).
    """
    lib = _loader.require_library()
    x = grad_q if grad_q is not None else grad_k
    if x is None:
        raise RuntimeError("rope_norm_bwd needs grad_q or grad_k")
    code, vec = _DTYPES[x.dtype]
    grad_q, grad_k = _strided(grad_q, vec, "grad_q"), _strided(grad_k, vec, "grad_k")
    q, k = _strided(q, vec, "q"), _strided(k, vec, "k")
    b, length, d = x.shape[0], x.shape[1], x.shape[3]
    tables = cos is not None or sin is not None
    if tables:
        cos, sin = (t.to(device=x.device, dtype=x.dtype).contiguous() for t in (cos, sin))
        pos, n_axes = None, 1
    else:
        pos, n_axes = _positions(positions, b, length)
    # (the gradients take their operands' strides: head-major views give head-major results)
    dq = torch.empty_like(grad_q) if grad_q is not None else None
    dk = torch.empty_like(grad_k) if grad_k is not None else None
    weights = []
    for t, w in ((grad_q, q_norm_weight), (grad_k, k_norm_weight)):
        weights.append(w.detach().to(device=x.device, dtype=torch.float32).contiguous()
                       if (w is not None and t is not None) else None)
    ts = None if tables else rope_timescale(d, max_wavelength, x.device)
    p = _loader.RopeNormBwdParams()
    p.dq_out, p.dk_out, p.q, p.k, p.dq, p.dk = _t4(grad_q), _t4(grad_k), _t4(q), _t4(k), _t4(dq), _t4(dk)
    if tables:
        p.cos, p.sin = cos.data_ptr(), sin.data_ptr()
    else:
        p.positions, p.timescale = pos.data_ptr(), ts.data_ptr()
    p.q_norm_weight = weights[0].data_ptr() if weights[0] is not None else None
    p.k_norm_weight = weights[1].data_ptr() if weights[1] is not None else None
    p.B, p.L, p.D = b, length, d
    p.H = grad_q.shape[2] if grad_q is not None else 0
    p.Hkv = grad_k.shape[2] if grad_k is not None else 0
    p.n_axes, p.dtype, p.norm_kind, p.norm_eps = n_axes, code, _NORM_KINDS[norm_kind], float(norm_eps)
    blocks = int(lib.bcattn_rope_norm_bwd_blocks(ctypes.byref(p)))
    partial = torch.empty((max(blocks, 1), 2, d), dtype=torch.float32, device=x.device)
    p.dw_partial = partial.data_ptr()
    with _on_device(x.device):
        _check(lib.bcattn_rope_norm_bwd(ctypes.byref(p), _stream(x.device)), lib)
    dw = partial[:blocks].sum(0)  # (2, D): one fixed-order reduction for both weights
    if stacked:
        return dq, dk, dw
    return dq, dk, (dw[0] if weights[0] is not None else None), (dw[1] if weights[1] is not None else None)


# The differentiable / traceable forms are torch.library ops (like the attention calls), so that
# ``torch.compile`` traces through them with the fake implementations and autograd sees the
# registered backward.  The rotation is orthogonal: its gradient is the rotation by minus the angle.
@torch.library.custom_op("bcattn::rope", mutates_args=())
def _op_rope(x: torch.Tensor, positions: torch.Tensor, max_wavelength: float, inverse: bool) -> torch.Tensor:
    return rope_raw(x, None, positions, max_wavelength, inverse=inverse)[0]


@_op_rope.register_fake
def _(x, positions, max_wavelength, inverse):
    return x.new_empty(x.shape)


@torch.library.custom_op("bcattn::rope_qk", mutates_args=())
def _op_rope_qk(q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor, max_wavelength: float,
                inverse: bool) -> tuple[torch.Tensor, torch.Tensor]:
    return rope_raw(q, k, positions, max_wavelength, inverse=inverse)


@_op_rope_qk.register_fake
def _(q, k, positions, max_wavelength, inverse):
    return q.new_empty(q.shape), k.new_empty(k.shape)


def _rope_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[-3])
    ctx.max_wavelength, ctx.inverse = inputs[-2], inputs[-1]


def _rope_backward(ctx, grad):
    (positions,) = ctx.saved_tensors
    return _op_rope(grad.contiguous(), positions, ctx.max_wavelength, not ctx.inverse), None, None, None


def _rope_qk_backward(ctx, grad_q, grad_k):
    (positions,) = ctx.saved_tensors
    dq, dk = _op_rope_qk(grad_q.contiguous(), grad_k.contiguous(), positions, ctx.max_wavelength, not ctx.inverse)
    return dq, dk, None, None, None


_op_rope.register_autograd(_rope_backward, setup_context=_rope_setup)
_op_rope_qk.register_autograd(_rope_qk_backward, setup_context=_rope_setup)


@torch.library.custom_op("bcattn::rope_tables", mutates_args=())
def _op_rope_tables(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                    inverse: bool) -> tuple[torch.Tensor, torch.Tensor]:
    return _rope_tables_bhsd(q, k, cos, sin, inverse=inverse)


@_op_rope_tables.register_fake
def _(q, k, cos, sin, inverse):
    return q.new_empty(q.shape), k.new_empty(k.shape)


def _rope_tables_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[2], inputs[3])
    ctx.inverse = inputs[4]


def _rope_tables_backward(ctx, grad_q, grad_k):
    cos, sin = ctx.saved_tensors
    dq, dk = _op_rope_tables(grad_q.contiguous(), grad_k.contiguous(), cos, sin, not ctx.inverse)
    return dq, dk, None, None, None


_op_rope_tables.register_autograd(_rope_tables_backward, setup_context=_rope_tables_setup)


# The forms with a per-head norm in front (q_norm / k_norm then the rotation): forward and gradient are
# one launch each.  layout 0: (B, L, H, D) operands, angles from positions, Gemma-3's norm
# (pi06/gemma3_with_expert.py:851-861); layout 1: (B, H, S, D) operands, cos / sin tables, the expert's
# norm (cosmos3/qwen3vl_with_expert.py:217-224).
def _norm_call(layout: int):
    return ((lambda t: t), "gemma3") if layout == 0 else ((lambda t: t.transpose(1, 2)), "qwen3")


@torch.library.custom_op("bcattn::rope_norm_qk", mutates_args=())
def _op_rope_norm_qk(q: torch.Tensor, k: torch.Tensor, angles_a: torch.Tensor, angles_b: torch.Tensor,
                     q_w: torch.Tensor, k_w: torch.Tensor, max_wavelength: float, eps: float,
                     layout: int) -> tuple[torch.Tensor, torch.Tensor]:
    view, kind = _norm_call(layout)
    qo, ko = torch.empty_like(q), torch.empty_like(k)
    kw = {"cos": angles_a, "sin": angles_b} if layout == 1 else {}
    rope_raw(view(q), view(k), None if layout == 1 else angles_a, max_wavelength, q_out=view(qo), k_out=view(ko),
             q_norm_weight=q_w, k_norm_weight=k_w, norm_eps=eps, norm_kind=kind, **kw)
    return qo, ko


@_op_rope_norm_qk.register_fake
def _(q, k, angles_a, angles_b, q_w, k_w, max_wavelength, eps, layout):
    return torch.empty_like(q), torch.empty_like(k)


@torch.library.custom_op("bcattn::rope_norm_qk_bwd", mutates_args=())
def _op_rope_norm_qk_bwd(grad_q: torch.Tensor, grad_k: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                         angles_a: torch.Tensor, angles_b: torch.Tensor, q_w: torch.Tensor, k_w: torch.Tensor,
                         max_wavelength: float, eps: float,
                         layout: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    view, kind = _norm_call(layout)
    kw = {"cos": angles_a, "sin": angles_b} if layout == 1 else {}
    dq, dk, dw = rope_norm_bwd_raw(view(grad_q), view(grad_k), view(q), view(k), None if layout == 1 else angles_a,
                                   max_wavelength, q_norm_weight=q_w, k_norm_weight=k_w, norm_eps=eps, norm_kind=kind,
                                   stacked=True, **kw)
    if layout == 1:  # (B, S, H, D) results of head-major operands: hand back head-major tensors
        dq, dk = view(dq).contiguous(), view(dk).contiguous()
    return dq, dk, dw


@_op_rope_norm_qk_bwd.register_fake
def _(grad_q, grad_k, q, k, angles_a, angles_b, q_w, k_w, max_wavelength, eps, layout):
    return torch.empty_like(q), torch.empty_like(k), q_w.new_empty((2, q.shape[-1]), dtype=torch.float32)


def _rope_norm_setup(ctx, inputs, output):
    q, k, angles_a, angles_b, q_w, k_w, max_wavelength, eps, layout = inputs
    ctx.save_for_backward(q, k, angles_a, angles_b, q_w, k_w)
    ctx.consts = (max_wavelength, eps, layout)


def _rope_norm_backward(ctx, grad_q, grad_k):
    q, k, angles_a, angles_b, q_w, k_w = ctx.saved_tensors
    dq, dk, dw = _op_rope_norm_qk_bwd(grad_q.contiguous(), grad_k.contiguous(), q, k, angles_a, angles_b,
                                      q_w, k_w, *ctx.consts)
    return dq, dk, None, None, dw[0].to(q_w.dtype), dw[1].to(k_w.dtype), None, None, None


_op_rope_norm_qk.register_autograd(_rope_norm_backward, setup_context=_rope_norm_setup)


def _rope_tables_bhsd(q, k, cos, sin, *, inverse=False, q_norm_weight=None, k_norm_weight=None, norm_eps=1e-6):
    """``q (B, H, S, D)``, ``k (B, Hkv, S, D)`` -> rotated tensors of the same shape (new storage)."""
    qo = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    ko = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    rope_raw(q.transpose(1, 2), k.transpose(1, 2), None, q_out=qo.transpose(1, 2), k_out=ko.transpose(1, 2),
             cos=cos, sin=sin, inverse=inverse, q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight,
             norm_eps=norm_eps, norm_kind="qwen3")
    return qo, ko


def _needs_graph(*ts: torch.Tensor) -> bool:
    return torch.compiler.is_compiling() or (torch.is_grad_enabled() and any(t.requires_grad for t in ts))


def apply_rope(x: torch.Tensor, positions: torch.Tensor, max_wavelength: float = 10_000) -> torch.Tensor:
    """``x (B, L, H, D)``, ``positions (B, L)`` or ``(A, B, L)`` -> rotated ``x``, same dtype.

    Drop-in for ``apply_rope`` of ``src/opentau/policies/pi05/paligemma_with_expert.py:52-107``:
    fp32 arithmetic, one rounding to ``x.dtype``; with 3-D positions band ``i`` follows axis
    ``i % A`` (interleaved MRoPE).  Differentiable in ``x``.
    """
    if _needs_graph(x):
        return _op_rope(x, positions, float(max_wavelength), False)
    return rope_raw(x, None, positions, max_wavelength)[0]


def apply_rope_qk(
    q: torch.Tensor,
    k: torch.Tensor,
    positions: torch.Tensor,
    max_wavelength: float = 10_000,
    *,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    norm_eps: float = 1e-6,
    q_out: torch.Tensor | None = None,
    k_out: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Both ``apply_rope`` calls of a layer (``paligemma_with_expert.py:739-740``) in one launch.

    With norm weights: ``apply_rope(q_norm(q), ...)`` and ``apply_rope(k_norm(k), ...)`` of
    ``src/opentau/policies/pi06/gemma3_with_expert.py:851-861`` where the norms are Gemma-3's
    (``x * rsqrt(mean(x^2) + eps) * (1 + weight)``, rounded to ``x.dtype``); differentiable in ``q``,
    ``k`` and both weights (one more launch for all four gradients).  ``q_out`` / ``k_out`` may be the inputs themselves (in place) or views of
    other storage, e.g. ``cache_k[:, n0:n0 + L]`` of a preallocated key cache.
    """
    norm = q_norm_weight is not None or k_norm_weight is not None
    if _needs_graph(q, k, *(w for w in (q_norm_weight, k_norm_weight) if w is not None)):
        if q_out is not None or k_out is not None:
            raise RuntimeError("apply_rope_qk is differentiable / traceable only without output arguments")
        if norm:
            if q_norm_weight is None or k_norm_weight is None:
                raise RuntimeError("the differentiable form takes both norm weights (or neither)")
            return _op_rope_norm_qk(q, k, positions, positions, q_norm_weight, k_norm_weight, float(max_wavelength),
                                    float(norm_eps), 0)
        return _op_rope_qk(q, k, positions, float(max_wavelength), False)
    return rope_raw(q, k, positions, max_wavelength, q_out=q_out, k_out=k_out, q_norm_weight=q_norm_weight,
                    k_norm_weight=k_norm_weight, norm_eps=norm_eps)


def apply_rotary_pos_emb(
    q: torch.Tensor,
    k: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    unsqueeze_dim: int = 1,
    *,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    norm_eps: float = 1e-6,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``q * cos + rotate_half(q) * sin`` (and the same for ``k``) in one launch.

    Signature and numerics of the ``apply_rotary_pos_emb`` that cosmos3's expert imports from
    ``transformers`` (``src/opentau/policies/cosmos3/qwen3vl_with_expert.py:70``, called ``:224``):
    ``cos`` / ``sin`` are ``(B, S, D)`` in the tensors' dtype, ``q`` / ``k`` are ``(B, H, S, D)`` with
    ``unsqueeze_dim=1`` (the expert's layout) or ``(B, S, H, D)`` with ``unsqueeze_dim=2``; every product
    and sum is rounded to that dtype.  Differentiable in ``q`` and ``k``.  With norm weights the expert's
    per-head RMS norm (``ExpertRMSNorm``, ``:85-102``) runs in front, i.e. ``:217-224`` in one call,
    differentiable in ``q``, ``k`` and the weights.
    """
    if unsqueeze_dim not in (1, 2):
        raise RuntimeError("unsqueeze_dim must be 1 (B, H, S, D) or 2 (B, S, H, D)")
    if unsqueeze_dim == 2:
        q, k = q.transpose(1, 2), k.transpose(1, 2)
    norm = q_norm_weight is not None or k_norm_weight is not None
    if _needs_graph(q, k, *(w for w in (q_norm_weight, k_norm_weight) if w is not None)):
        if norm:
            if q_norm_weight is None or k_norm_weight is None:
                raise RuntimeError("the differentiable form takes both norm weights (or neither)")
            qo, ko = _op_rope_norm_qk(q, k, cos, sin, q_norm_weight, k_norm_weight, 0.0, float(norm_eps), 1)
        else:
            qo, ko = _op_rope_tables(q, k, cos, sin, False)
    else:
        qo, ko = _rope_tables_bhsd(q, k, cos, sin, q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight,
                                   norm_eps=norm_eps)
    if unsqueeze_dim == 2:
        qo, ko = qo.transpose(1, 2), ko.transpose(1, 2)
    return qo, ko
