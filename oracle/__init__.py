"""CPU oracle for the SAE decoder-loss path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped ``flexsae_amd`` package never
does (it fails loudly when its HIP library is missing instead of falling back).

Three independent statements of the same two closed forms live here:

* :func:`loss_grads` -- the plain-C restatement in ``sae_oracle.c`` (double
  accumulation, analytic gradients from the definition, OpenMP over D slices).
* :func:`brute_force` -- pure-Python/numpy loops straight from the definition,
  for tiny shapes only.
* :func:`torch_loss` -- a torch restatement of the reference's pure-torch
  definitions (reference ``torch-ext/flex_sae/hierarchical_kernels.py:312-323``
  and ``torch-ext/flex_sae/topk_kernels.py:226-237``) whose gradients come from
  ``torch.autograd`` rather than from any hand derivation; chunkable over B.
  This is also what the benchmark times as the CPU baseline.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsae_oracle.so")
_lib = None

TOPK = 0
HIER = 1


def build(force: bool = False) -> str:
    """Compile ``sae_oracle.c`` with gcc (``make``) and return the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libsae_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, dbl = ctypes.c_int64, ctypes.c_double
    p = ctypes.c_void_p
    lib.sae_oracle_loss_grads.restype = ctypes.c_int
    lib.sae_oracle_loss_grads.argtypes = [ctypes.c_int, p, p, p, p, p, i64, i64, i64, i64, dbl,
                                          p, p, p, p, p]
    lib.sae_oracle_csr.restype = ctypes.c_int
    lib.sae_oracle_csr.argtypes = [p, i64, i64, i64, p, p]
    lib.sae_oracle_max_threads.restype = ctypes.c_int
    _lib = lib
    return lib


def max_threads() -> int:
    return int(load().sae_oracle_max_threads())


def _as_f32(x) -> np.ndarray:
    """Exact upcast of a torch tensor / array (fp32, bf16, fp16) to contiguous float32."""
    try:
        import torch

        if isinstance(x, torch.Tensor):
            x = x.detach().to("cpu").to(torch.float32).numpy()
    except ImportError:  # pragma: no cover
        pass
    return np.ascontiguousarray(x, dtype=np.float32)


def _as_i64(x) -> np.ndarray:
    try:
        import torch

        if isinstance(x, torch.Tensor):
            x = x.detach().to("cpu").numpy()
    except ImportError:  # pragma: no cover
        pass
    return np.ascontiguousarray(x, dtype=np.int64)


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def loss_grads(mode: int, indices, weight, vals, bias, target, grad_out: float = 1.0,
               want_dw: bool = True, dw_float32: bool = False, want_grads: bool = True):
    """Loss and gradients from the C oracle.

    Returns ``(loss, dW, dvals, dbias)`` as python float / numpy arrays (float64,
    or float32 for dW when ``dw_float32``); the gradients are already multiplied
    by ``grad_out``.  Missing pieces are ``None``.
    """
    lib = load()
    idx = _as_i64(indices)
    W, v, b, t = _as_f32(weight), _as_f32(vals), _as_f32(bias), _as_f32(target)
    B, K = idx.shape
    F, D = W.shape
    assert v.shape == (B, K) and b.shape == (D,) and t.shape == (B, D)
    loss = np.zeros(1, dtype=np.float64)
    dW = dW32 = dv = db = None
    if want_grads:
        dv = np.zeros((B, K), dtype=np.float64)
        db = np.zeros((D,), dtype=np.float64)
        if want_dw:
            if dw_float32:
                dW32 = np.zeros((F, D), dtype=np.float32)
            else:
                dW = np.zeros((F, D), dtype=np.float64)
    rc = lib.sae_oracle_loss_grads(int(mode), _ptr(idx), _ptr(W), _ptr(v), _ptr(b), _ptr(t),
                                   B, K, F, D, float(grad_out), _ptr(loss), _ptr(dW), _ptr(dW32),
                                   _ptr(dv), _ptr(db))
    if rc != 0:
        raise ValueError(f"sae_oracle_loss_grads failed with code {rc}")
    return float(loss[0]), (dW32 if dw_float32 else dW), dv, db


def csr(indices, F: int):
    """Stable latent-major pair list: ``begin[F+1]`` and ``map[B*K]`` (both uint32)."""
    lib = load()
    idx = _as_i64(indices)
    B, K = idx.shape
    begin = np.zeros(F + 1, dtype=np.uint32)
    mp = np.zeros(B * K, dtype=np.uint32)
    rc = lib.sae_oracle_csr(_ptr(idx), B, K, int(F), _ptr(begin), _ptr(mp))
    if rc != 0:
        raise ValueError(f"sae_oracle_csr failed with code {rc}")
    return begin, mp


def brute_force(mode: int, indices, weight, vals, bias, target, grad_out: float = 1.0):
    """Definition-level loops in float64 (tiny shapes only): every prefix
    reconstruction is rebuilt from scratch, gradients by the chain rule on the
    materialised ``[B,K,D]`` residuals."""
    idx = _as_i64(indices)
    W = _as_f32(weight).astype(np.float64)
    v = _as_f32(vals).astype(np.float64)
    bia = _as_f32(bias).astype(np.float64)
    t = _as_f32(target).astype(np.float64)
    B, K = idx.shape
    F, D = W.shape
    steps = range(K) if mode == HIER else [K - 1]
    n_terms = B * len(steps) * D
    loss = 0.0
    dW = np.zeros_like(W)
    dv = np.zeros_like(v)
    db = np.zeros_like(bia)
    for b in range(B):
        for k in steps:
            for d in range(D):
                r = bia[d]
                for j in range(k + 1):
                    r += v[b, j] * W[idx[b, j], d]
                diff = r - t[b, d]
                loss += diff * diff
                gd = 2.0 * diff / n_terms * grad_out
                db[d] += gd
                for j in range(k + 1):
                    dv[b, j] += gd * W[idx[b, j], d]
                    dW[idx[b, j], d] += gd * v[b, j]
    return loss / n_terms, dW, dv, db


def torch_loss(mode: int, indices, weight, vals, bias, target, compute_dtype=None,
               chunk_rows: Optional[int] = None):
    """Torch restatement of the reference's pure-torch definitions.

    gather rows -> scale by vals -> sum (TopK) or cumsum (Hierarchical) over K ->
    add bias, subtract target -> mean of squares.  ``compute_dtype`` defaults to
    float32 like the reference's ``.to(torch.float32)`` casts; pass
    ``torch.float64`` for an autograd ground truth.  With ``chunk_rows`` the batch
    is processed in slices and the partial sums of squares are added, which is
    the same value up to summation order and keeps ``[Bc,K,D]`` small.
    """
    import torch

    cd = compute_dtype or torch.float32
    B, K = indices.shape
    D = weight.shape[1]
    step = chunk_rows or B
    total = None
    for b0 in range(0, B, step):
        sl = slice(b0, min(B, b0 + step))
        rows = weight[indices[sl]].to(cd)
        scaled = rows * vals[sl].to(cd).unsqueeze(-1)
        if mode == HIER:
            recon = bias.to(cd) + scaled.cumsum(dim=1)
            diff = recon - target[sl].to(cd).unsqueeze(1)
        else:
            recon = bias.to(cd) + scaled.sum(dim=1)
            diff = recon - target[sl].to(cd)
        part = diff.pow(2).sum()
        total = part if total is None else total + part
    denom = B * D * (K if mode == HIER else 1)
    return total / denom
