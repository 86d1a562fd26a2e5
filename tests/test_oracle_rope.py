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
