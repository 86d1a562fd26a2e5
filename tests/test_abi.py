"""Host-side checks that need no GPU: the C-ABI library loads, exports every
symbol the header declares, and the Python surface fails loudly without a GPU."""

import ctypes
import re
import subprocess
from pathlib import Path

import pytest
import torch

from opentau_amd import attention, flash_attn_hip
from opentau_amd.flash_attn_hip import _loader

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "bcattn.h"


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(bcattn_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_bound_entry_points():
    assert _declared_functions() == sorted(_loader.EXPORTS)


def test_library_loads_and_exports_every_declared_symbol():
    lib = _loader.load_library()
    for name in _declared_functions():
        assert hasattr(lib, name), name
    assert lib.bcattn_abi_version() == _loader.ABI_VERSION


def test_struct_layout_matches_header(tmp_path):
    """Sizes and field offsets of the ctypes mirrors against what a C compiler makes of include/bcattn.h."""
    fields = {
        "bcattn_tensor": (_loader.Tensor4, ["ptr", "stride_b", "stride_s", "stride_h"]),
        "bcattn_fwd_params": (_loader.FwdParams, [f[0] for f in _loader.FwdParams._fields_]),
        "bcattn_bwd_params": (_loader.BwdParams, [f[0] for f in _loader.BwdParams._fields_]),
        "bcattn_rope_params": (_loader.RopeParams, [f[0] for f in _loader.RopeParams._fields_]),
        "bcattn_rope_norm_bwd_params": (_loader.RopeNormBwdParams, [f[0] for f in _loader.RopeNormBwdParams._fields_]),
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "bcattn.h"', "int main(void) {"]
    for cname, (_, names) in fields.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        lines += [f'  printf("{cname}.{n} %zu\\n", offsetof({cname}, {n}));' for n in names]
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", str(ROOT / "include"), "-o", str(exe), str(src)], check=True)
    want = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True,
                                                        text=True).stdout.splitlines())
    assert ctypes.sizeof(_loader.Tensor4) == 32
    for cname, (ctype, names) in fields.items():
        assert ctypes.sizeof(ctype) == int(want[cname]), cname
        for n in names:
            assert getattr(ctype, n).offset == int(want[f"{cname}.{n}"]), f"{cname}.{n}"


def test_workspace_queries_run_without_a_gpu():
    lib = _loader.load_library()
    p = _loader.FwdParams()
    p.B, p.Sq, p.Sk0, p.Sk1, p.H, p.Hkv, p.D, p.dtype = 8, 50, 968, 50, 8, 1, 256, _loader.DTYPE_BF16
    fwd = lib.bcattn_fwd_workspace_bytes(ctypes.byref(p))
    kvc = lib.bcattn_fwd_kvcache_workspace_bytes(ctypes.byref(p))
    # 16 + 1 key tiles per sample (the two segments are tiled separately): a 16-byte summary
    # and 64 merged ids per tile, each array rounded up to 256 bytes
    assert fwd == (8 * 17 * 16 + 255) // 256 * 256 + 8 * 17 * 64 * 4
    assert kvc > fwd
    bp = _loader.BwdParams()
    bp.B, bp.Sq, bp.Sk, bp.H, bp.Hkv, bp.D = 2, 100, 130, 4, 2, 128
    assert lib.bcattn_bwd_workspace_bytes(ctypes.byref(bp)) >= 2 * 4 * 100 * 4
    # One sample, one kv head: the 8 key blocks' dK/dV work is shared out over the 8 query heads, and the
    # workspace grows by the fp32 partial sums, 2 (dK, dV) x 8 x Sk x D floats; with 8 kv heads (no groups
    # to share out) it does not.
    bp.B, bp.Sq, bp.Sk, bp.H, bp.Hkv, bp.D, bp.dtype = 1, 1024, 1024, 8, 1, 256, _loader.DTYPE_BF16
    shared = lib.bcattn_bwd_workspace_bytes(ctypes.byref(bp))
    bp.Hkv = 8
    assert shared - lib.bcattn_bwd_workspace_bytes(ctypes.byref(bp)) == 2 * 8 * 1024 * 256 * 4


def test_argument_errors_are_reported_not_crashed():
    lib = _loader.load_library()
    p = _loader.FwdParams()
    assert lib.bcattn_fwd(ctypes.byref(p), None) == _loader.ERR_INVALID
    assert b"shape" in lib.bcattn_last_error()
    p.B, p.Sq, p.Sk0, p.H, p.Hkv, p.D, p.dtype, p.scale = 1, 4, 4, 3, 2, 128, 1, 1.0
    assert lib.bcattn_fwd(ctypes.byref(p), None) == _loader.ERR_INVALID
    assert b"multiple" in lib.bcattn_last_error()
    p.H = 4
    p.D = 80
    assert lib.bcattn_fwd(ctypes.byref(p), None) == _loader.ERR_UNSUPPORTED
    assert b"head_dim" in lib.bcattn_last_error()
    p.D, p.dtype = 128, 7
    assert lib.bcattn_fwd(ctypes.byref(p), None) == _loader.ERR_UNSUPPORTED
    p.dtype = 1
    assert lib.bcattn_fwd(ctypes.byref(p), None) == _loader.ERR_INVALID  # null q
    assert b"null" in lib.bcattn_last_error()
    assert lib.bcattn_bwd(None, None) == _loader.ERR_INVALID
    # the gradient of the norm + rotary call: argument checks come before anything touches a device
    assert lib.bcattn_rope_norm_bwd(None, None) == _loader.ERR_INVALID
    r = _loader.RopeNormBwdParams()
    r.B, r.L, r.H, r.Hkv, r.D, r.n_axes, r.dtype = 1, 4, 2, 1, 96, 1, _loader.DTYPE_BF16
    assert lib.bcattn_rope_norm_bwd(ctypes.byref(r), None) == _loader.ERR_UNSUPPORTED
    assert b"power-of-two" in lib.bcattn_last_error()
    r.D = 128
    assert lib.bcattn_rope_norm_bwd(ctypes.byref(r), None) == _loader.ERR_INVALID  # no positions / tables
    assert lib.bcattn_rope_norm_bwd_blocks(ctypes.byref(r)) == 0  # (no gradient tensors: nothing to launch)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU behaviour")
def test_no_fallback_without_gpu():
    _loader._reset_for_tests()
    assert flash_attn_hip.is_available() is False
    assert "HIP device" in flash_attn_hip.load_error()
    q = torch.zeros(1, 4, 2, 64)
    ids = flash_attn_hip.make_att_block_ids(torch.ones(1, 4, dtype=torch.bool), torch.zeros(1, 4))
    with pytest.raises(RuntimeError, match="unavailable"):
        flash_attn_hip.flash_attn_blockmask(q, q, q, *ids, 0.125)
    with pytest.raises(RuntimeError, match="unavailable"):
        attention.flash_attention_forward(None, ids, 1, 64, q, q, q)


def test_kill_switch(monkeypatch):
    monkeypatch.setenv("OPENTAU_DISABLE_FLASH_HIP", "1")
    with pytest.raises(RuntimeError, match="disabled"):
        _loader.load_library()


def test_build_attention_inputs_contract():
    pad = torch.ones(2, 6, dtype=torch.bool)
    att = torch.tensor([[0, 0, 1, 0, 1, 1]] * 2)
    mask, ids = attention.build_attention_inputs(True, pad, att)
    assert mask is None and len(ids) == 4
    assert ids[0].tolist()[0] == [0, 0, 1, 1, 2, 3]
    cross_pad = torch.ones(2, 3, dtype=torch.bool)
    _, ids = attention.build_attention_inputs(True, pad, att, 3, cross_pad)
    assert ids[1].shape == (2, 9) and int(ids[1][0, 0]) == flash_attn_hip.INT_BLK_MIN
    with pytest.raises(RuntimeError):
        attention.build_attention_inputs(False, pad, att)
    with pytest.raises(ValueError):
        flash_attn_hip.make_att_block_ids(pad[0], att)
    with pytest.raises(AssertionError):
        flash_attn_hip.make_att_block_ids(pad, att, 3, None)


def test_fake_impl_gives_shapes_without_running_kernels():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        q = torch.empty(2, 50, 8, 256, dtype=torch.bfloat16)
        k = torch.empty(2, 90, 1, 256, dtype=torch.bfloat16)
        ids = (torch.empty(2, 50, dtype=torch.int32), torch.empty(2, 90, dtype=torch.int32),
               torch.empty(2, 50, dtype=torch.bool), torch.empty(2, 90, dtype=torch.bool))
        out, lse = torch.ops.bcattn.fwd(q, k, k, *ids, 0.0625)
        assert out.shape == (2, 50, 8, 256) and out.dtype == torch.bfloat16
        assert lse.shape == (2, 8, 50) and lse.dtype == torch.float32
        dq, dk, dv = torch.ops.bcattn.bwd(out, q, k, k, out, lse, *ids, 0.0625)
        assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == k.shape
        import opentau_amd.rope  # noqa: F401  (registers the rotary ops)

        pos = torch.empty(2, 50, dtype=torch.long)
        rq, rk = torch.ops.bcattn.rope_qk(q, k[:, :50], pos, 10000.0, False)
        assert rq.shape == q.shape and rk.shape == (2, 50, 1, 256) and rk.dtype == torch.bfloat16
        assert torch.ops.bcattn.rope(q, pos, 10000.0, True).shape == q.shape
        qh, cs = q.transpose(1, 2), torch.empty(2, 50, 256, dtype=torch.bfloat16)
        tq, tk = torch.ops.bcattn.rope_tables(qh, qh[:, :1], cs, cs, False)
        assert tq.shape == qh.shape and tk.shape == (2, 1, 50, 256)


def test_workloads_are_seeded_and_shaped():
    from opentau_amd.workloads import make_workload

    w = make_workload("c1")
    assert w.q.shape == (1, 354, 8, 256) and w.k.shape == (1, 354, 1, 256) and w.q.dtype == torch.float32
    assert w.pairs() == 304 * 304 + 50 * 354
    w2 = make_workload("c1")
    assert torch.equal(w.q, w2.q) and torch.equal(w.v, w2.v)
    w3 = make_workload("c3", batch=2)
    n = 512 + w3.text_len
    exp = int((n * n + 64 * n + 2080 + 50 * (n + 114)).sum())
    assert w3.pairs() == exp


def test_bench_refuses_more_than_one_gpu():
    """One GPU is all this build drives: ``bench.py --gpus N`` with N > 1 says so and exits."""
    import subprocess
    import sys

    root = Path(__file__).resolve().parent.parent
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_entry_points_exist():
    import importlib.util

    root = Path(__file__).resolve().parent.parent
    spec = importlib.util.spec_from_file_location("graft_entry", root / "__graft_entry__.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert callable(mod.build) and callable(mod.smoke)
