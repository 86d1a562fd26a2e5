"""The reference harness's long-context point (``src/opentau/scripts/benchmark_flash_attn.py:329-388``:
B1 H8 Hkv1 D256, prefix-LM mask -- first half one block, second half strictly causal -- up to S = 98 304)
at full size.  A dense oracle cannot run there (the mask alone is 9.7 GB, the fp32 scores 309 GB), so:

* sampled query rows are checked against the eager oracle, which for a subset of the rows needs only
  ``(rows, S)`` scores: O and dQ of a row depend on nothing but that row's q, dO and all keys;
* dV and dK, which need every row, are held to two identities of the backward: the rows of P sum to
  one, so ``sum_j dV[j] = sum over heads and valid rows of dO``; and ``sum_j dS[i, j] = 0`` for every
  row, so ``sum_j dK[j] = 0``.
"""

import pytest
import torch

from opentau_amd import flash_attn_hip as fa
from oracle import eager

from helpers import assert_close_bf16, randn, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_kernels():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    if not fa.is_available():
        raise RuntimeError(f"HIP kernels unavailable on a GPU box: {fa.load_error()}")


def _harness_ids(b, s):
    att = torch.zeros(b, s, dtype=torch.int32)
    att[:, s // 2:] = 1  # benchmark_flash_attn.py:76-85, pattern "prefixlm"
    return fa.make_att_block_ids(torch.ones(b, s, dtype=torch.bool), att)


def test_reference_sweep_end_point_98304():
    b, s, h, hkv, d = 1, 98304, 8, 1, 256
    scale = d**-0.5
    ids = _harness_ids(b, s)
    gen = torch.Generator(device=DEV).manual_seed(11)
    q, go = (torch.randn(b, s, h, d, generator=gen, device=DEV, dtype=torch.float32).bfloat16() for _ in range(2))
    k, v = (torch.randn(b, s, hkv, d, generator=gen, device=DEV, dtype=torch.float32).bfloat16() for _ in range(2))
    gi = [t.to(DEV) for t in ids]
    out, lse = fa.forward_raw(q, k, v, *gi, scale)
    dq, dk, dv = fa.backward_raw(go, q, k, v, out, lse, *gi, scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(dq.float()).all()

    # sampled rows against the eager oracle (on the CPU): first and last rows of either half, tile
    # edges, and a few in between
    rows = torch.tensor(sorted({0, 1, 63, 64, 4097, s // 2 - 1, s // 2, s // 2 + 1, s // 2 + 64, 3 * s // 4 + 5,
                                s - 65, s - 2, s - 1}))
    kc, vc = k.cpu(), v.cpu()
    qs, gos = q[:, rows.to(DEV)].cpu(), go[:, rows.to(DEV)].cpu()
    sub_ids = (ids[0][:, rows], ids[1], ids[2][:, rows], ids[3])
    ro, rq, _, _ = eager.eager_grads(qs, kc, vc, gos, *sub_ids, scale)
    assert_close_bf16(out[:, rows.to(DEV)].cpu().float(), ro.float(), "O, sampled rows")
    got_dq = dq[:, rows.to(DEV)].cpu().float()
    assert rel_l2(got_dq, rq.float()) <= 1e-2, rel_l2(got_dq, rq.float())
    # a causal row's LSE: the first causal row sees the whole first half and itself
    ref_lse = eager.attention_lse(qs, kc, *sub_ids, scale)
    torch.testing.assert_close(lse[:, :, rows.to(DEV)].cpu(), ref_lse, atol=2e-3, rtol=2e-3)

    # identities over all rows
    dv_sum, want = dv.float().sum(1), go.float().sum(1).reshape(b, hkv, h // hkv, d).sum(2)
    assert rel_l2(dv_sum, want) <= 1e-2, rel_l2(dv_sum, want)
    # sum_j dK[j] = 0: against the size of what cancels
    dk_sum, dk_abs = dk.float().sum(1).abs().max(), dk.float().abs().sum(1).max()
    assert float(dk_sum / dk_abs) <= 2e-3, float(dk_sum / dk_abs)


@pytest.mark.parametrize("b,s", [(2, 512), (2, 768), (1, 1024), (1, 2048)])
def test_reference_harness_shapes_fwd_bwd(b, s):
    """The four shapes the reference's harness times (``benchmark_flash_attn.py:405``), H8 Hkv1 D256, prefix-LM
    mask, forward + backward through the op against the eager oracle."""
    h, hkv, d = 8, 1, 256
    scale = d**-0.5
    ids = _harness_ids(b, s)
    q, k, v, go = (randn(sh, torch.bfloat16, 70 + n) for n, sh in enumerate(
        [(b, s, h, d), (b, s, hkv, d), (b, s, hkv, d), (b, s, h, d)]))
    ro, rq, rk, rv = eager.eager_grads(q, k, v, go, *ids, scale)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = fa.flash_attn_blockmask(qg, kg, vg, *[t.to(DEV) for t in ids], scale)
    out.backward(go.to(DEV))
    torch.cuda.synchronize()
    for name, got, ref in (("out", out.detach(), ro), ("dq", qg.grad, rq), ("dk", kg.grad, rk), ("dv", vg.grad, rv)):
        r = rel_l2(got.cpu().float(), ref.float())
        assert r <= 1e-2, (name, r)
