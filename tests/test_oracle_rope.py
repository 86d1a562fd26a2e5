"""Pins of the rotary-embedding oracle (CPU only)."""

import torch

from oracle import rope
from tests.helpers import randn, rel_l2


def test_reference_shape_and_dtype_preserved():
    # the reference's tests/policies/test_pi06.py:159-164
    x = randn((2, 4, 3, 32), torch.float32, 0)
    positions = torch.arange(4)[None, :].expand(2, 4)
    out = rope.apply_rope(x, positions, max_wavelength=10_000.0)
    assert out.shape == x.shape and out.dtype == x.dtype
    assert rope.apply_rope(x.bfloat16(), positions).dtype == torch.bfloat16


def test_reference_different_thetas_differ():
    # tests/policies/test_pi06.py:166-172
    x = randn((1, 8, 2, 16), torch.float32, 1)
    positions = torch.arange(8)[None, :]
    assert not torch.allclose(rope.apply_rope(x, positions, 10_000.0), rope.apply_rope(x, positions, 1_000_000.0))


def test_reference_position_zero_is_identity():
    # tests/policies/test_pi06.py:174-180
    x = torch.ones(1, 1, 1, 8)
    out = rope.apply_rope(x, torch.zeros(1, 1, dtype=torch.long), 10_000.0)
    assert torch.allclose(out, x, atol=1e-6)


def test_known_answers():
    # D = 2: one band of timescale 1, so (1, 0) at position p becomes (cos p, sin p)
    x = torch.tensor([1.0, 0.0]).reshape(1, 1, 1, 2).expand(1, 3, 1, 2)
    p = torch.tensor([[0, 1, 2]])
    out = rope.apply_rope(x, p)
    want = torch.stack([torch.cos(p[0].float()), torch.sin(p[0].float())], -1).reshape(1, 3, 1, 2)
    assert torch.allclose(out, want, atol=1e-6)
    # D = 4, wavelength 10000: band 1 has timescale 10000 ** (2/4) = 100
    x = torch.tensor([0.0, 1.0, 0.0, 0.0]).reshape(1, 1, 1, 4)
    out = rope.apply_rope(x, torch.tensor([[50]]))
    assert torch.allclose(out.flatten(), torch.tensor([0.0, 0.87758256, 0.0, 0.47942554]), atol=1e-6)


def test_closed_form_complex_rotation():
    x = randn((2, 5, 3, 16), torch.float32, 2)
    positions = torch.tensor([[0, 1, 2, 7, 30], [3, 3, 4, 11, 49]])
    for w in (10_000, 1_000_000):
        want = rope.rope_closed_form(x, positions, w)
        assert rel_l2(rope.apply_rope(x, positions, w), want) <= 1e-6


def test_rotation_keeps_pair_norms_and_composes():
    x = randn((2, 6, 2, 32), torch.float32, 3)
    p = torch.randint(0, 40, (2, 6), generator=torch.Generator().manual_seed(0))
    q = torch.randint(0, 40, (2, 6), generator=torch.Generator().manual_seed(1))
    y = rope.apply_rope(x, p)
    n = lambda t: t[..., :16] ** 2 + t[..., 16:] ** 2  # noqa: E731
    assert torch.allclose(n(y), n(x), rtol=1e-5, atol=1e-6)
    assert rel_l2(rope.apply_rope(y, q), rope.apply_rope(x, p + q)) <= 1e-5


def test_mrope_equal_axes_is_plain_rope_bit_for_bit():
    x = randn((2, 7, 2, 64), torch.bfloat16, 4)
    p = torch.randint(0, 500, (2, 7), generator=torch.Generator().manual_seed(2))
    assert torch.equal(rope.apply_rope(x, p), rope.apply_rope(x, p[None].expand(3, 2, 7)))


def test_mrope_band_follows_axis_i_mod_a():
    x = randn((1, 4, 2, 16), torch.float32, 5)
    p3 = torch.randint(0, 30, (3, 1, 4), generator=torch.Generator().manual_seed(3))
    assert rel_l2(rope.apply_rope(x, p3), rope.rope_closed_form(x, p3)) <= 1e-6
    # and it matters: moving the axes changes the result
    assert not torch.allclose(rope.apply_rope(x, p3), rope.apply_rope(x, p3.flip(0)))


def test_gemma3_rms_norm_closed_form_and_special_cases():
    x = randn((2, 3, 4, 64), torch.float32, 6)
    w = randn((64,), torch.float32, 7) * 0.1
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * (1.0 + w.double())
    assert rel_l2(rope.gemma3_rms_norm(x, w), want) <= 1e-6
    unit = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    assert torch.allclose(rope.gemma3_rms_norm(unit, torch.zeros(64)), unit, atol=1e-5)
    assert torch.allclose(rope.gemma3_rms_norm(8.0 * x, w), rope.gemma3_rms_norm(x, w), atol=1e-5)
    assert rope.gemma3_rms_norm(x.bfloat16(), w.bfloat16()).dtype == torch.bfloat16


def test_rotary_tables_form_equals_apply_rope_in_fp32_and_the_closed_form():
    x = randn((2, 6, 3, 32), torch.float32, 8)
    k = randn((2, 6, 1, 32), torch.float32, 9)
    p = torch.randint(0, 40, (2, 6), generator=torch.Generator().manual_seed(4))
    cos, sin = rope.rope_tables(p, 32)
    qo, ko = rope.apply_rotary_pos_emb(x, k, cos, sin, unsqueeze_dim=2)
    assert rel_l2(qo, rope.apply_rope(x, p)) <= 1e-6 and rel_l2(ko, rope.apply_rope(k, p)) <= 1e-6
    assert rel_l2(qo, rope.rope_closed_form(x, p)) <= 1e-6
    # head-major layout, unsqueeze_dim = 1
    qh, kh = rope.apply_rotary_pos_emb(x.transpose(1, 2), k.transpose(1, 2), cos, sin)
    assert torch.equal(qh.transpose(1, 2), qo) and torch.equal(kh.transpose(1, 2), ko)


def test_rotary_tables_form_against_the_library_routine():
    m = __import__("pytest").importorskip("transformers.models.qwen3_vl.modeling_qwen3_vl")
    for dtype in (torch.bfloat16, torch.float32):
        q, k = randn((2, 4, 7, 64), dtype, 10), randn((2, 2, 7, 64), dtype, 11)
        p = torch.randint(0, 900, (2, 7), generator=torch.Generator().manual_seed(5))
        cos, sin = rope.rope_tables(p, 64, 1_000_000, dtype)
        want = m.apply_rotary_pos_emb(q, k, cos, sin)
        got = rope.apply_rotary_pos_emb(q, k, cos, sin)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_rotary_tables_form_rounds_every_step_in_bf16():
    bf = torch.bfloat16
    x = torch.tensor([257.0, 3.0]).to(bf).reshape(1, 1, 1, 2)       # 257 -> 256 in bf16 (8 significant bits)
    cos = torch.tensor([[[1.5, 1.5]]]).to(bf)
    sin = torch.tensor([[[0.75, 0.75]]]).to(bf)
    out, _ = rope.apply_rotary_pos_emb(x, x, cos, sin, unsqueeze_dim=2)
    # first element: bf16(256 * 1.5) + bf16(-3 * 0.75) = 384 + (-2.25) = 381.75 -> bf16 382
    # second: bf16(3 * 1.5) + bf16(256 * 0.75) = 4.5 + 192 = 196.5 -> bf16 196 (tie to even) ... exact sums
    assert out.flatten().tolist() == [382.0, 196.0]
    # a case where the separately rounded product matters: 1.0078125 * 1.0078125 = 1.01568... -> bf16 1.015625;
    # 0.00390625 added after gives 1.01953125, a tie that goes to the even 1.015625, whereas the exact sum
    # 1.01959... rounded once goes up to 1.0234375
    x = torch.tensor([1.0078125, 0.00390625]).to(bf).reshape(1, 1, 1, 2)
    cos = torch.tensor([[[1.0078125, 1.0]]]).to(bf)
    sin = torch.tensor([[[-1.0, 0.0]]]).to(bf)
    out, _ = rope.apply_rotary_pos_emb(x, x, cos, sin, unsqueeze_dim=2)
    once = torch.tensor(1.0078125 * 1.0078125 + 0.00390625).to(bf)
    assert float(out[0, 0, 0, 0]) == 1.015625 and float(once) == 1.0234375


def test_expert_rms_norm_closed_form_and_roundings():
    x = randn((2, 3, 4, 64), torch.float32, 12)
    w = 1.0 + randn((64,), torch.float32, 13) * 0.1
    xd = x.double()
    want = w.double() * (xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6))
    assert rel_l2(rope.expert_rms_norm(x, w), want) <= 1e-6
    unit = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    assert torch.allclose(rope.expert_rms_norm(unit, torch.ones(64)), unit, atol=1e-5)
    # bf16: the normalised value is rounded before it meets the weight
    xb, wb = x.bfloat16(), w.bfloat16()
    xf = xb.float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    assert torch.equal(rope.expert_rms_norm(xb, wb), (wb.float() * normed.float()).bfloat16())
    assert rope.expert_rms_norm(xb, w).dtype == torch.bfloat16  # fp32 weight on a bf16 input


def _forward64(kind, x, w, angle):
    """Norm then rotation in float64, written out: ``x (..., D)``, ``angle (..., D/2)``."""
    half = x.shape[-1] // 2
    r = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    y = x * r * ((1.0 + w) if kind == "gemma3" else w)
    lo, hi = y[..., :half], y[..., half:]
    c, s = torch.cos(angle), torch.sin(angle)
    return torch.cat([lo * c - hi * s, hi * c + lo * s], -1)


def test_norm_rope_gradients_against_finite_differences():
    """The gradient the fused backward is held to: autograd through the oracle's norm and rotation, checked
    here against central differences of a float64 restatement of the forward (which the forward tests
    above tie to the oracle).  A dropped mean term, a wrong sign of the inverse rotation or a missing
    ``1 +`` on Gemma-3's weight each fail it."""
    b, length, h, d = 2, 5, 3, 32
    pos = torch.randint(0, 50, (b, length), generator=torch.Generator().manual_seed(1))
    x = randn((b, length, h, d), torch.float32, 2) * 1.5
    w = randn((d,), torch.float32, 3) * 0.3
    go = randn((b, length, h, d), torch.float32, 4)
    timescale = 10_000.0 ** ((2.0 / d) * torch.arange(d // 2, dtype=torch.float64))
    angle = (pos.double().unsqueeze(-1) / timescale).unsqueeze(-2)  # (B, L, 1, D/2)
    cos, sin = rope.rope_tables(pos, d, 10_000)
    picks = torch.randint(0, x.numel(), (24,), generator=torch.Generator().manual_seed(5)).tolist()
    for kind in ("gemma3", "qwen3"):
        wk = w if kind == "gemma3" else 1.0 + w
        if kind == "gemma3":
            fwd = rope.apply_rope(rope.gemma3_rms_norm(x, wk), pos)
            dx, dw = rope.norm_rope_backward(x, wk, go, kind=kind, positions=pos)
        else:
            xt, gt = x.transpose(1, 2).contiguous(), go.transpose(1, 2).contiguous()
            fwd = rope.apply_rotary_pos_emb(rope.expert_rms_norm(xt, wk), xt[:, :0], cos, sin)[0].transpose(1, 2)
            dx, dw = rope.norm_rope_backward(xt, wk, gt, kind=kind, cos=cos, sin=sin)
            dx = dx.transpose(1, 2)
        assert rel_l2(fwd, _forward64(kind, x.double(), wk.double(), angle)) <= 1e-6

        def loss(xv, wv):
            return float((_forward64(kind, xv, wv, angle) * go.double()).sum())

        step = 1e-6
        for at in picks:
            e = torch.zeros(x.numel(), dtype=torch.float64)
            e[at] = step
            e = e.view_as(x)
            fd = (loss(x.double() + e, wk.double()) - loss(x.double() - e, wk.double())) / (2 * step)
            assert abs(fd - float(dx.flatten()[at])) <= 2e-4 * max(1.0, abs(fd)), (kind, at, fd)
        for at in range(0, d, 5):
            e = torch.zeros(d, dtype=torch.float64)
            e[at] = step
            fd = (loss(x.double(), wk.double() + e) - loss(x.double(), wk.double() - e)) / (2 * step)
            assert abs(fd - float(dw[at])) <= 2e-4 * max(1.0, abs(fd)), (kind, "w", at, fd)
