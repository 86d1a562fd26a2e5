"""Pins the CPU oracle (oracle/eager.py) before anything is checked against it:
known answers restated from the reference's own tests, a library routine (SDPA),
an independent float64 brute force (oracle/bcattn_ref.c), closed-form special
cases and gradcheck.  No GPU."""

import pytest
import torch

from helpers import PATTERNS, att_masks, make_blocks, randn, rel_l2
from opentau_amd.flash_attn_hip import INT_BLK_MIN, make_att_block_ids
from oracle import bruteforce, eager


# ---- make_att_2d_masks: known answers (reference tests/policies/test_pi06.py:62-152) ----
def test_mask_bidirectional_all_true():
    pad = torch.ones(1, 4, dtype=torch.bool)
    att = torch.zeros(1, 4, dtype=torch.int32)
    assert eager.make_att_2d_masks(pad, att).all()


def test_mask_causal_is_tril():
    pad = torch.ones(1, 6, dtype=torch.bool)
    att = torch.ones(1, 6, dtype=torch.int32)
    assert torch.equal(eager.make_att_2d_masks(pad, att)[0], torch.tril(torch.ones(6, 6)).bool())


def test_mask_prefix_lm():
    pad = torch.ones(1, 6, dtype=torch.bool)
    att = torch.tensor([[0, 0, 0, 1, 1, 1]], dtype=torch.int32)
    m = eager.make_att_2d_masks(pad, att)[0]
    exp = torch.tensor(
        [[1, 1, 1, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 0],
         [1, 1, 1, 1, 1, 1]]
    ).bool()
    assert torch.equal(m, exp)


def test_mask_four_blocks_docstring_example():
    # [[1 0 1 0 1 0 0 1 0 0]]: causal between 4 blocks (modeling_pi05.py:138-139)
    att = torch.tensor([[1, 0, 1, 0, 1, 0, 0, 1, 0, 0]], dtype=torch.int32)
    pad = torch.ones(1, 10, dtype=torch.bool)
    m = eager.make_att_2d_masks(pad, att)[0]
    blk = [0, 0, 1, 1, 2, 2, 2, 3, 3, 3]
    for i in range(10):
        for j in range(10):
            assert bool(m[i, j]) == (blk[j] <= blk[i])


def test_mask_padding_kills_rows_and_cols():
    pad = torch.tensor([[True, True, False, True]])
    att = torch.zeros(1, 4, dtype=torch.int32)
    m = eager.make_att_2d_masks(pad, att)[0]
    assert not m[2].any() and not m[:, 2].any()
    assert m[[0, 1, 3]][:, [0, 1, 3]].all()


def test_mask_cross_block_prepended():
    pad = torch.tensor([[True, True]])
    att = torch.tensor([[1, 1]], dtype=torch.int32)
    cross_pad = torch.tensor([[True, False, True]])
    m = eager.make_att_2d_masks(pad, att, n_cross_att_tokens=3, cross_att_pad_masks=cross_pad)
    assert m.shape == (1, 2, 5)
    exp = torch.tensor([[[1, 0, 1, 1, 0], [1, 0, 1, 1, 1]]]).bool()
    assert torch.equal(m, exp)


def test_mask_bf16_att_masks():
    # the suffix att mask is built in the embedding dtype (modeling_pi05.py:1633)
    pad = torch.ones(2, 7, dtype=torch.bool)
    att = torch.tensor([[1, 0, 0, 1, 0, 1, 1]] * 2)
    a = eager.make_att_2d_masks(pad, att.to(torch.bfloat16))
    b = eager.make_att_2d_masks(pad, att.to(torch.int32))
    assert torch.equal(a, b)


def test_mask_bruteforce_loop():
    g = torch.Generator().manual_seed(0)
    pad = torch.rand(3, 13, generator=g) > 0.25
    att = (torch.rand(3, 13, generator=g) > 0.6).to(torch.int32)
    cpad = torch.rand(3, 5, generator=g) > 0.3
    m = eager.make_att_2d_masks(pad, att, 5, cpad)
    for b in range(3):
        cum = 0
        cums = []
        for t in range(13):
            cum += int(att[b, t])
            cums.append(cum)
        for i in range(13):
            for j in range(5):
                assert bool(m[b, i, j]) == bool(pad[b, i] and cpad[b, j])
            for j in range(13):
                assert bool(m[b, i, 5 + j]) == bool(pad[b, i] and pad[b, j] and cums[j] <= cums[i])


def test_mask_rejects_non_2d():
    with pytest.raises(ValueError):
        eager.make_att_2d_masks(torch.ones(4, dtype=torch.bool), torch.zeros(1, 4))
    with pytest.raises(ValueError):
        eager.make_att_2d_masks(torch.ones(1, 4, dtype=torch.bool), torch.zeros(4))


# ---- block ids == dense mask (reference tests/policies/test_flash_attn_cuda.py:94-117) ----
@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_block_ids_reconstruct_dense_mask(pattern, impl):
    fn = eager.make_att_block_ids if impl == "oracle" else make_att_block_ids
    b, n = 3, 24
    pad = torch.ones(b, n, dtype=torch.bool)
    pad[0, -4:] = False
    att = att_masks(pattern, b, n)
    ids = fn(pad, att)
    assert ids[0].dtype == torch.int32 and ids[2].dtype == torch.bool
    assert torch.equal(eager.dense_mask_from_block_ids(*ids), eager.make_att_2d_masks(pad, att))


@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_block_ids_reconstruct_cross_attention_mask(impl):
    fn = eager.make_att_block_ids if impl == "oracle" else make_att_block_ids
    b, n, cross = 2, 16, 10
    pad = torch.ones(b, n, dtype=torch.bool)
    pad[0, -3:] = False
    att = att_masks("causal", b, n)
    cross_pad = torch.ones(b, cross, dtype=torch.bool)
    cross_pad[1, -2:] = False
    ids = fn(pad, att, cross, cross_pad)
    ref = eager.make_att_2d_masks(pad, att, n_cross_att_tokens=cross, cross_att_pad_masks=cross_pad)
    recon = eager.dense_mask_from_block_ids(*ids)
    assert recon.shape == ref.shape == (b, n, cross + n)
    assert torch.equal(recon, ref)
    assert int(ids[1][0, 0]) == INT_BLK_MIN


def test_product_block_ids_equal_oracle_on_random_masks():
    g = torch.Generator().manual_seed(5)
    for _ in range(5):
        pad = torch.rand(4, 37, generator=g) > 0.2
        att = (torch.rand(4, 37, generator=g) > 0.7).to(torch.int32)
        cp = torch.rand(4, 9, generator=g) > 0.2
        for a, b in zip(make_att_block_ids(pad, att, 9, cp), eager.make_att_block_ids(pad, att, 9, cp)):
            assert torch.equal(a, b)


# ---- eager attention vs the library routine (reference tests/policies/test_pi0.py:209-254) ----
@pytest.mark.parametrize("h,hkv,d,s", [(4, 2, 16, 16), (4, 4, 16, 16), (8, 1, 64, 40)])
def test_eager_matches_sdpa_fp32(h, hkv, d, s):
    b = 2
    q, k, v = randn((b, s, h, d), torch.float32, 1), randn((b, s, hkv, d), torch.float32, 2), randn(
        (b, s, hkv, d), torch.float32, 3)
    pad = torch.ones(b, s, dtype=torch.bool)
    att = att_masks("prefixlm", b, s)
    mask = eager.make_att_2d_masks(pad, att)
    out_e = eager.eager_attention_bshd(mask, q, k, v)
    out_s = eager.sdpa_attention_bshd(mask, q, k, v)
    assert out_e.shape == (b, s, h * d)
    torch.testing.assert_close(out_e, out_s, atol=1e-4, rtol=1e-4)


def test_eager_pure_causal_matches_is_causal_sdpa():
    b, s, h, d = 2, 19, 4, 32
    q, k, v = (randn((b, s, h, d), torch.float32, i) for i in (4, 5, 6))
    mask = eager.make_att_2d_masks(torch.ones(b, s, dtype=torch.bool), torch.ones(b, s, dtype=torch.int32))
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True
    ).transpose(1, 2).reshape(b, s, h * d)
    torch.testing.assert_close(eager.eager_attention_bshd(mask, q, k, v), ref, atol=1e-5, rtol=1e-5)


def test_eager_bhsd_equals_bshd():
    b, s, h, hkv, d = 2, 23, 8, 2, 32
    q, k, v = randn((b, s, h, d), torch.float32, 7), randn((b, s, hkv, d), torch.float32, 8), randn(
        (b, s, hkv, d), torch.float32, 9)
    ids = make_blocks(b, s, "multiblock", pad_tail=3)
    mask = eager.dense_mask_from_block_ids(*ids)
    o1 = eager.eager_attention_bshd(mask, q, k, v)
    o2 = eager.eager_attention_bhsd(mask, q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
    valid = ids[2][:, :, None]
    torch.testing.assert_close(o1 * valid, o2 * valid, atol=1e-6, rtol=1e-6)


def test_eager_scaling_kwarg():
    b, s, h, d = 1, 9, 2, 16
    q, k, v = (randn((b, s, h, d), torch.float32, i) for i in (1, 2, 3))
    mask = torch.ones(b, s, s, dtype=torch.bool)
    a = eager.eager_attention_bshd(mask, q, k, v, scaling=0.37)
    ref = torch.softmax(torch.einsum("bqhd,bkhd->bhqk", q, k) * 0.37, -1)
    ref = torch.einsum("bhqk,bkhd->bqhd", ref, v).reshape(b, s, h * d)
    torch.testing.assert_close(a, ref, atol=1e-5, rtol=1e-5)


def test_eager_single_visible_key_returns_that_value():
    b, s, h, d = 1, 6, 2, 8
    q, k, v = (randn((b, s, h, d), torch.float32, i) for i in (1, 2, 3))
    mask = torch.zeros(b, s, s, dtype=torch.bool)
    for i in range(s):
        mask[0, i, (i * 2) % s] = True
    out = eager.eager_attention_bshd(mask, q, k, v).reshape(b, s, h, d)
    for i in range(s):
        torch.testing.assert_close(out[0, i], v[0, (i * 2) % s])


def test_eager_equal_keys_give_mean_of_visible_values():
    b, s, h, d = 1, 8, 2, 8
    q, v = randn((b, s, h, d), torch.float32, 1), randn((b, s, h, d), torch.float32, 3)
    k = torch.ones(b, s, h, d)
    ids = make_blocks(b, s, "causal")
    out = eager.eager_attention_bshd(eager.dense_mask_from_block_ids(*ids), q, k, v).reshape(b, s, h, d)
    for i in range(s):
        torch.testing.assert_close(out[0, i], v[0, : i + 1].mean(0), atol=1e-6, rtol=1e-5)


def test_eager_padded_row_is_uniform_mean():
    # fully masked rows: every score equals the fill value, softmax is uniform
    b, s, h, d = 1, 5, 1, 4
    q, k, v = (randn((b, s, h, d), torch.float32, i) for i in (1, 2, 3))
    mask = torch.ones(b, s, s, dtype=torch.bool)
    mask[0, 2] = False
    out = eager.eager_attention_bshd(mask, q, k, v).reshape(b, s, h, d)
    torch.testing.assert_close(out[0, 2], v[0].mean(0), atol=1e-6, rtol=1e-5)


def test_eager_bf16_cast_order():
    # probabilities are rounded to bf16 before P@V; scores are computed in fp32
    b, s, h, d = 1, 12, 2, 16
    q, k, v = (randn((b, s, h, d), torch.bfloat16, i) for i in (1, 2, 3))
    mask = torch.ones(b, s, s, dtype=torch.bool)
    out = eager.eager_attention_bshd(mask, q, k, v)
    assert out.dtype == torch.bfloat16
    p = torch.softmax(torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float()) * d**-0.5, -1).to(torch.bfloat16)
    ref = torch.matmul(p, v.permute(0, 2, 1, 3)).permute(0, 2, 1, 3).reshape(b, s, h * d)
    assert torch.equal(out, ref)


# ---- eager / reference / lse vs the float64 brute force in C ----
@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("hkv", [1, 2])
def test_eager_matches_bruteforce(pattern, hkv):
    b, s, h, d = 2, 21, 4, 32
    q, k, v = randn((b, s, h, d), torch.float32, 1), randn((b, s, hkv, d), torch.float32, 2), randn(
        (b, s, hkv, d), torch.float32, 3)
    ids = make_blocks(b, s, pattern, pad_tail=3, pad_mid=(4, 7))
    scale = d**-0.5
    bo, blse = bruteforce.fwd(q, k, v, *ids, scale)
    eo = eager.eager_from_block_ids(q, k, v, *ids, scale)
    ro, has = eager.reference_attention_fp32(q, k, v, *ids, scale)
    valid = ids[2][:, :, None, None]
    assert rel_l2(eo * valid, bo * valid) < 1e-6
    assert rel_l2(ro, bo) < 1e-6
    assert torch.equal(has, ids[2])  # every valid row sees itself
    lse = eager.attention_lse(q, k, *ids, scale)
    assert rel_l2(lse, blse) < 1e-6


def test_cross_layout_matches_bruteforce():
    b, sq, h, hkv, d, cross = 2, 33, 8, 1, 64, 20
    ids = make_blocks(b, sq, "causal", cross=cross)
    q = randn((b, sq, h, d), torch.float32, 1)
    k = randn((b, cross + sq, hkv, d), torch.float32, 2)
    v = randn((b, cross + sq, hkv, d), torch.float32, 3)
    bo, _ = bruteforce.fwd(q, k, v, *ids, d**-0.5)
    eo = eager.eager_from_block_ids(q, k, v, *ids, d**-0.5)
    assert rel_l2(eo, bo) < 1e-6


def test_lse_rows_sum_to_one():
    b, s, h, d = 2, 17, 2, 16
    q, k = randn((b, s, h, d), torch.float32, 1), randn((b, s, h, d), torch.float32, 2)
    ids = make_blocks(b, s, "multiblock", pad_tail=2)
    scale = 0.25
    lse = eager.attention_lse(q, k, *ids, scale)
    scores = torch.einsum("bqhd,bkhd->bhqk", q, k) * scale
    mask = eager.dense_mask_from_block_ids(*ids)[:, None]
    p = torch.where(mask, torch.exp(scores - lse[..., None]), torch.zeros(()))
    rows = p.sum(-1)
    exp = ids[2][:, None, :].expand_as(rows).float()
    torch.testing.assert_close(rows, exp, atol=1e-5, rtol=1e-5)
    assert (lse.transpose(1, 2)[~ids[2]] == 0).all()


# ---- backward ----
@pytest.mark.parametrize("pattern", ["causal", "prefixlm", "multiblock"])
def test_eager_grads_match_bruteforce(pattern):
    b, s, h, hkv, d = 2, 18, 4, 2, 16
    q, k, v = randn((b, s, h, d), torch.float32, 1), randn((b, s, hkv, d), torch.float32, 2), randn(
        (b, s, hkv, d), torch.float32, 3)
    go = randn((b, s, h, d), torch.float32, 4)
    ids = make_blocks(b, s, pattern, pad_tail=2)
    scale = d**-0.5
    _, dq, dk, dv = eager.eager_grads(q, k, v, go, *ids, scale)
    bq, bk, bv = bruteforce.bwd(q, k, v, go * ids[2][:, :, None, None], *ids, scale)
    qm = ids[2][:, :, None, None]
    assert rel_l2(dq * qm, bq) < 1e-5
    assert rel_l2(dk, bk) < 1e-5
    assert rel_l2(dv, bv) < 1e-5


def test_eager_gradcheck_float64():
    b, s, h, hkv, d = 1, 6, 2, 1, 4
    g = torch.Generator().manual_seed(0)
    q = torch.randn(b, s, h, d, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(b, s, hkv, d, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(b, s, hkv, d, generator=g, dtype=torch.float64, requires_grad=True)
    ids = make_blocks(b, s, "prefixlm")
    mask = eager.dense_mask_from_block_ids(*ids)

    def fn(q, k, v):
        # float64 statement of the same formula (the oracle itself upcasts to fp32)
        kk = k.repeat_interleave(h // hkv, dim=2)
        vv = v.repeat_interleave(h // hkv, dim=2)
        w = torch.einsum("bqhd,bkhd->bhqk", q, kk) * d**-0.5
        w = torch.where(mask[:, None], w, torch.full((), eager.BIG_NEG, dtype=torch.float64))
        return torch.einsum("bhqk,bkhd->bqhd", torch.softmax(w, -1), vv)

    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-5)
    out64 = fn(q, k, v).detach()
    out32 = eager.eager_from_block_ids(q.detach().float(), k.detach().float(), v.detach().float(), *ids, d**-0.5)
    assert rel_l2(out32, out64) < 1e-6


# ---- the float64 model of a flash kernel's rounding points ----
@pytest.mark.parametrize("pattern", ["causal", "prefixlm", "multiblock"])
def test_flash_rounding_model_without_rounding_is_the_closed_form(pattern):
    """With every rounding off the model is the textbook backward: pinned by the float64 brute force
    (an independent C routine) and by autograd through the eager oracle."""
    from oracle import flash_rounding

    b, s, h, hkv, d = 2, 18, 4, 2, 16
    q, k, v = randn((b, s, h, d), torch.float32, 1), randn((b, s, hkv, d), torch.float32, 2), randn(
        (b, s, hkv, d), torch.float32, 3)
    go = randn((b, s, h, d), torch.float32, 4)
    ids = make_blocks(b, s, pattern, pad_tail=2)
    scale = d**-0.5
    o, dq, dk, dv = flash_rounding.flash_grads_rounded(q, k, v, go, *ids, scale)
    qm = ids[2][:, :, None, None]
    bo, _ = bruteforce.fwd(q, k, v, *ids, scale)
    bq, bk, bv = bruteforce.bwd(q, k, v, go * qm, *ids, scale)
    assert rel_l2(o * qm, bo * qm) < 1e-12
    assert rel_l2(dq, bq) < 1e-12 and rel_l2(dk, bk) < 1e-12 and rel_l2(dv, bv) < 1e-12
    _, eq, ek, ev = eager.eager_grads(q, k, v, go, *ids, scale)
    assert rel_l2(eq * qm, dq) < 1e-5 and rel_l2(ek, dk) < 1e-5 and rel_l2(ev, dv) < 1e-5


def test_flash_rounding_model_rounds_where_it_says():
    """One query row, one dominant key: dK is the small difference P * (dP - delta).  Rounding O (hence
    delta) to bf16 moves dK by far more than rounding dS does; with the roundings off the bf16 inputs
    give the exact closed form.  (This is the arithmetic behind the single-row GPU cases.)"""
    from oracle import flash_rounding

    b, h, hkv, d, sk = 3, 2, 1, 64, 41
    q = (randn((b, 1, h, d), torch.float32, 11) * 3).to(torch.bfloat16)
    k, v, go = (randn((b, sk, hkv, d), torch.bfloat16, 12), randn((b, sk, hkv, d), torch.bfloat16, 13),
                randn((b, 1, h, d), torch.bfloat16, 14))
    ids = make_att_block_ids(torch.ones(b, 1, dtype=torch.bool), torch.ones(b, 1, dtype=torch.int32), sk - 1,
                             torch.ones(b, sk - 1, dtype=torch.bool))
    scale = d**-0.5
    exact = flash_rounding.flash_grads_rounded(q, k, v, go, *ids, scale, round_o=False, round_p=False, round_ds=False)
    bq, bk, bv = bruteforce.bwd(q.float(), k.float(), v.float(), go.float(), *ids, scale)
    assert rel_l2(exact[2], bk) < 1e-12 and rel_l2(exact[1], bq) < 1e-12 and rel_l2(exact[3], bv) < 1e-12
    only_o = flash_rounding.flash_grads_rounded(q, k, v, go, *ids, scale, round_p=False, round_ds=False)
    only_ds = flash_rounding.flash_grads_rounded(q, k, v, go, *ids, scale, round_o=False, round_p=False)
    err_o, err_ds = rel_l2(only_o[2], exact[2]), rel_l2(only_ds[2], exact[2])
    assert 0 < err_ds < 2e-3 < err_o < 3e-2, (err_ds, err_o)
    assert rel_l2(only_o[3], exact[3]) == 0.0  # dV does not see delta
