"""ctypes binding of ``bcattn_ref.c`` (float64 brute force). Test infrastructure only."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np
import torch

_DIR = Path(__file__).resolve().parent
_LIB = None


def build() -> Path:
    subprocess.run(["make", "-s", "-C", str(_DIR)], check=True)
    return _DIR / "libbcattn_ref.so"


def _lib():
    global _LIB
    if _LIB is None:
        so = _DIR / "libbcattn_ref.so"
        if not so.exists():
            build()
        _LIB = ctypes.CDLL(str(so))
    return _LIB


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _prep(q, k, v, q_blk, k_blk, q_valid, k_valid):
    f = lambda t: np.ascontiguousarray(t.detach().float().cpu().numpy())  # noqa: E731
    i = lambda t: np.ascontiguousarray(t.cpu().numpy().astype(np.int32))  # noqa: E731
    u = lambda t: np.ascontiguousarray(t.cpu().numpy().astype(np.uint8))  # noqa: E731
    return f(q), f(k), f(v), i(q_blk), i(k_blk), u(q_valid), u(k_valid)


def fwd(q, k, v, q_blk, k_blk, q_valid, k_valid, scale):
    """Returns ``(out (B,Sq,H,D) float64, lse (B,H,Sq) float64)`` as torch tensors."""
    qa, ka, va, qb, kb, qv, kv = _prep(q, k, v, q_blk, k_blk, q_valid, k_valid)
    b, sq, h, d = qa.shape
    sk, hkv = ka.shape[1], ka.shape[2]
    out = np.zeros((b, sq, h, d), np.float64)
    lse = np.zeros((b, h, sq), np.float64)
    rc = _lib().bcref_fwd(_p(qa), _p(ka), _p(va), _p(qb), _p(kb), _p(qv), _p(kv), b, sq, sk, h, hkv, d,
                          ctypes.c_double(scale), _p(out), _p(lse))
    assert rc == 0, rc
    return torch.from_numpy(out), torch.from_numpy(lse)


def bwd(q, k, v, d_out, q_blk, k_blk, q_valid, k_valid, scale):
    """Returns ``(dq, dk, dv)`` float64."""
    qa, ka, va, qb, kb, qv, kv = _prep(q, k, v, q_blk, k_blk, q_valid, k_valid)
    do = np.ascontiguousarray(d_out.detach().float().cpu().numpy())
    b, sq, h, d = qa.shape
    sk, hkv = ka.shape[1], ka.shape[2]
    dq = np.zeros((b, sq, h, d), np.float64)
    dk = np.zeros((b, sk, hkv, d), np.float64)
    dv = np.zeros((b, sk, hkv, d), np.float64)
    rc = _lib().bcref_bwd(_p(qa), _p(ka), _p(va), _p(do), _p(qb), _p(kb), _p(qv), _p(kv), b, sq, sk, h, hkv,
                          d, ctypes.c_double(scale), _p(dq), _p(dk), _p(dv))
    assert rc == 0, rc
    return torch.from_numpy(dq), torch.from_numpy(dk), torch.from_numpy(dv)
