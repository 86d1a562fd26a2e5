"""The committed fixtures of ``tests/golden`` (made once by the float64 brute force in C, see
``tests/golden/make_fixtures.py``) against the eager oracle on the CPU and against the HIP
kernels, in every element type, on the GPU.  The inputs are regenerated from their seeds."""

import importlib.util
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import eager

GOLDEN = Path(__file__).resolve().parent / "golden"
_spec = importlib.util.spec_from_file_location("make_fixtures", GOLDEN / "make_fixtures.py")
fixtures = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(fixtures)
NAMES = sorted(fixtures.CASES)


def _expected(name):
    with np.load(GOLDEN / f"{name}.npz") as z:
        return {k: torch.from_numpy(z[k]) for k in ("out", "lse", "dq", "dk", "dv")}


ROPE_NAMES = sorted(fixtures.ROPE_CASES)


def test_every_case_has_its_fixture():
    assert sorted(p.stem for p in GOLDEN.glob("*.npz")) == sorted(NAMES + ROPE_NAMES)


def _rope_expected(name):
    with np.load(GOLDEN / f"{name}.npz") as z:
        return torch.from_numpy(z["out"])


@pytest.mark.parametrize("name", ROPE_NAMES)
def test_rope_oracle_reproduces_the_fixtures(name):
    from oracle import rope as oracle_rope

    x, positions, w = fixtures.rope_inputs(name)
    assert rel_l2(oracle_rope.apply_rope(x, positions, w), _rope_expected(name)) <= 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,rel", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2), (torch.float16, 2e-3)])
@pytest.mark.parametrize("name", ROPE_NAMES)
def test_rope_kernel_reproduces_the_fixtures(name, dtype, rel):
    from opentau_amd import rope as hip_rope
    from oracle import rope as oracle_rope

    x, positions, w = fixtures.rope_inputs(name, dtype)
    # a 16-bit run is held to the closed form on the rounded inputs
    want = _rope_expected(name) if dtype == torch.float32 else oracle_rope.rope_closed_form(x.float(), positions, w)
    got = hip_rope.apply_rope(x.to("cuda:0"), positions.to("cuda:0"), w)
    assert got.dtype == dtype and rel_l2(got.float().cpu(), want) <= rel


@pytest.mark.parametrize("name", NAMES)
def test_eager_oracle_reproduces_the_fixtures(name):
    q, k, v, d_out, ids, scale = fixtures.case_inputs(name)
    want = _expected(name)
    out, dq, dk, dv = eager.eager_grads(q, k, v, d_out, *ids, scale)
    qm = ids[2][:, :, None, None]
    for got, key in ((out * qm, "out"), (dq * qm, "dq"), (dk, "dk"), (dv, "dv")):
        ref = want[key] * qm if key in ("out", "dq") else want[key]
        assert rel_l2(got, ref) <= 1e-5, key
    lse = eager.attention_lse(q, k, *ids, scale) * ids[2][:, None, :]
    torch.testing.assert_close(lse, want["lse"] * ids[2][:, None, :], atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,rel", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2), (torch.float16, 2e-3)])
@pytest.mark.parametrize("name", NAMES)
def test_kernels_reproduce_the_fixtures(name, dtype, rel):
    from opentau_amd import flash_attn_hip as fa

    assert fa.is_available(), f"flash_hip kernel unavailable: {fa.load_error()}"
    # the inputs are rounded to the element type first: the fixture of a 16-bit run is the
    # brute force on those rounded inputs
    q, k, v, d_out, ids, scale = fixtures.case_inputs(name, dtype)
    if dtype == torch.float32:
        want = _expected(name)
    else:
        from oracle import bruteforce

        o64, l64 = bruteforce.fwd(q.float(), k.float(), v.float(), *ids, scale)
        g64 = bruteforce.bwd(q.float(), k.float(), v.float(), d_out.float(), *ids, scale)
        want = dict(out=o64.float(), lse=l64.float(), dq=g64[0].float(), dk=g64[1].float(), dv=g64[2].float())
    dev = "cuda"
    gi = [t.to(dev) for t in ids]
    out, lse = fa.forward_raw(q.to(dev), k.to(dev), v.to(dev), *gi, scale)
    dq, dk, dv = fa.backward_raw(d_out.to(dev), q.to(dev), k.to(dev), v.to(dev), out, lse, *gi, scale)
    qm = ids[2][:, :, None, None]
    for got, key in ((out, "out"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        g = got.float().cpu()
        ref = want[key]
        if key in ("out", "dq"):
            g, ref = g * qm, ref * qm
        assert rel_l2(g, ref) <= rel, key
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    torch.testing.assert_close(lse.cpu() * ids[2][:, None, :], want["lse"] * ids[2][:, None, :], atol=tol, rtol=tol)
