"""Thin test-side callers of the C-ABI (include/flexsae_amd.h) on torch device tensors.

They allocate outputs/workspaces with torch and pass raw pointers, the way a foreign-language
binding would; return codes are handed back unchanged so tests can assert on them.
"""
import ctypes

import torch

from flexsae_amd import _lib

DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}


def ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def shape_of(indices, weight, vals, bias_dtype=torch.float32, target_dtype=torch.float32):
    B, K = indices.shape
    F, D = weight.shape
    return _lib.Shape(B, K, F, D, DT[weight.dtype], DT[vals.dtype], DT[bias_dtype], DT[target_dtype])


def forward(mode, indices, weight, vals, bias, target, flag=None):
    """mode 'hier' | 'topk' -> (rc, loss, resid)."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals, bias.dtype, target.dtype)
    dev = weight.device
    nbytes = lib.flexsae_fwd_workspace_bytes(ctypes.byref(sh))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=dev)
    resid = torch.full((sh.B, sh.D), float("nan"), dtype=torch.float32, device=dev)
    fn = lib.flexsae_hier_fwd if mode == "hier" else lib.flexsae_topk_fwd
    rc = fn(ctypes.byref(sh), ptr(indices), ptr(weight), ptr(vals), ptr(bias), ptr(target), ptr(loss),
            ptr(resid), ptr(ws), nbytes, ptr(flag), stream())
    return rc, loss, resid


def hier_backward(indices, weight, vals, resid, grad_out, flag=None, slice_cols=0, dw_dtype=torch.float32):
    """Two-phase backward -> (rc, dW in dw_dtype, dvals fp32, dbias fp32); `slice_cols` sets the
    workspace size (0 = the minimum, one tile per pass)."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals)
    dev = weight.device
    dW = torch.full((sh.F, sh.D), float("nan"), dtype=dw_dtype, device=dev)
    dv = torch.full((sh.B, sh.K), float("nan"), dtype=torch.float32, device=dev)
    db = torch.full((sh.D,), float("nan"), dtype=torch.float32, device=dev)
    g = torch.tensor([grad_out], dtype=torch.float32, device=dev)
    nbytes = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), slice_cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.flexsae_hier_bwd(ctypes.byref(sh), ptr(indices), ptr(weight), ptr(vals), ptr(resid), ptr(g),
                              ptr(dW), DT[dw_dtype], ptr(dv), ptr(db), ptr(ws), nbytes, 0, ptr(flag), stream())
    return rc, dW, dv, db


def hier_train(indices, weight, vals, bias, target, flag=None, slice_cols=0, dw_dtype=torch.float32, flags=0,
               alloc_dw=True, keep_workspace=False, workspace=None):
    """Fused forward+backward for a unit upstream gradient -> (rc, loss, dW, dvals, dbias);
    ``alloc_dw=False`` passes a null dW (for FLEXSAE_BWD_NO_DW); ``keep_workspace`` appends the
    workspace to the result (for flexsae_hier_hot_stats); ``workspace`` is one kept from an earlier
    call (for the reuse flags)."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals, bias.dtype, target.dtype)
    dev = weight.device
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=dev)
    dW = torch.full((sh.F, sh.D), float("nan"), dtype=dw_dtype, device=dev) if alloc_dw else None
    dv = torch.full((sh.B, sh.K), float("nan"), dtype=torch.float32, device=dev)
    db = torch.full((sh.D,), float("nan"), dtype=torch.float32, device=dev)
    # slices of whole training tiles where the entry point supports the shape
    nbytes = (lib.flexsae_hier_fwd_bwd_workspace_bytes_flags(ctypes.byref(sh), slice_cols, flags)
              or lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), slice_cols))
    ws = workspace if workspace is not None else torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    assert ws.numel() >= nbytes
    rc = lib.flexsae_hier_fwd_bwd(ctypes.byref(sh), ptr(indices), ptr(weight), ptr(vals), ptr(bias), ptr(target),
                                  ptr(loss), ptr(dW), DT[dw_dtype], ptr(dv), ptr(db), ptr(ws), nbytes, flags,
                                  ptr(flag), stream())
    if keep_workspace:
        return rc, loss, dW, dv, db, ws
    return rc, loss, dW, dv, db


def hot_stats(indices, weight, vals, bias, target, workspace):
    """flexsae_hier_hot_stats -> [hot latents, candidates, cold long latents, threshold, deferred walks]."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals, bias.dtype, target.dtype)
    stats = torch.zeros(5, dtype=torch.int32, device=weight.device)
    rc = lib.flexsae_hier_hot_stats(ctypes.byref(sh), ptr(workspace), ptr(stats), stream())
    assert rc == 0, _lib.status_string(rc)
    return [int(x) for x in stats.cpu()]


def hier_sgd_step(indices, weight, vals, bias, target, step, flag=None, slice_cols=0, flags=0):
    """Training step with the SGD update of ``weight`` fused in (in place) -> (rc, loss, dvals, dbias)."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals, bias.dtype, target.dtype)
    dev = weight.device
    loss = torch.full((1,), float("nan"), dtype=torch.float32, device=dev)
    dv = torch.full((sh.B, sh.K), float("nan"), dtype=torch.float32, device=dev)
    db = torch.full((sh.D,), float("nan"), dtype=torch.float32, device=dev)
    nbytes = lib.flexsae_hier_fwd_bwd_workspace_bytes_flags(ctypes.byref(sh), slice_cols, flags)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    st = torch.tensor([step], dtype=torch.float32, device=dev)
    rc = lib.flexsae_hier_sgd_step(ctypes.byref(sh), ptr(indices), ptr(weight), ptr(vals), ptr(bias), ptr(target),
                                   ptr(st), ptr(loss), ptr(dv), ptr(db), ptr(ws), nbytes, flags, ptr(flag), stream())
    return rc, loss, dv, db


def scale(src, g, in_place=False):
    lib = _lib.load()
    dst = src if in_place else torch.full_like(src, float("nan"))
    gt = torch.tensor([g], dtype=torch.float32, device=src.device)
    rc = lib.flexsae_scale(ptr(dst), ptr(src), DT[src.dtype], src.numel(), ptr(gt), stream())
    return rc, dst


def hier_backward_atomic(indices, weight, vals, resid, grad_out, flag=None, prezeroed=False):
    """Atomic fallback -> (rc, dW_acc fp32, dvals fp32, dbias fp32)."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals)
    dev = weight.device
    fill = 0.0 if prezeroed else float("nan")  # the entry point must zero-fill by itself
    dW = torch.full((sh.F, sh.D), fill, dtype=torch.float32, device=dev)
    dv = torch.full((sh.B, sh.K), fill, dtype=torch.float32, device=dev)
    db = torch.full((sh.D,), fill, dtype=torch.float32, device=dev)
    g = torch.tensor([grad_out], dtype=torch.float32, device=dev)
    rc = lib.flexsae_hier_bwd_atomic(ctypes.byref(sh), ptr(indices), ptr(weight), ptr(vals), ptr(resid),
                                     ptr(g), ptr(dW), ptr(dv), ptr(db),
                                     _lib.BWD_OUTPUTS_PREZEROED if prezeroed else 0, ptr(flag), stream())
    return rc, dW, dv, db


def csr_build(indices, F, flag=None):
    """-> (rc, begin int64 tensor [F+1], map int64 tensor [B*K]) (uint32 payloads widened)."""
    lib = _lib.load()
    B, K = indices.shape
    dev = indices.device
    begin = torch.full((F + 1,), -1, dtype=torch.int32, device=dev)
    mp = torch.full((B * K,), -1, dtype=torch.int32, device=dev)
    nbytes = lib.flexsae_csr_workspace_bytes(B, K, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.flexsae_csr_build(ptr(indices), B, K, F, ptr(begin), ptr(mp), ptr(ws), nbytes, ptr(flag),
                               stream())
    return rc, begin, mp


def widen_u32(t):
    return t.to(torch.int64) & 0xFFFFFFFF


def topk_backward(indices, weight, vals, resid, grad_out, dw_dtype=None, slice_cols=0, flags=0, pass_indices=True):
    """-> (rc, dW in dw_dtype, dvals fp32, dbias fp32); builds the pair list first."""
    lib = _lib.load()
    sh = shape_of(indices, weight, vals)
    dev = weight.device
    rc, begin, mp = csr_build(indices, sh.F)
    if rc != 0:
        return rc, None, None, None
    dw_dtype = dw_dtype or weight.dtype
    dW = torch.full((sh.F, sh.D), float("nan"), dtype=dw_dtype, device=dev)
    dv = torch.full((sh.B, sh.K), float("nan"), dtype=torch.float32, device=dev)
    db = torch.full((sh.D,), float("nan"), dtype=torch.float32, device=dev)
    g = torch.tensor([grad_out], dtype=torch.float32, device=dev)
    nbytes = lib.flexsae_topk_bwd_workspace_bytes(ctypes.byref(sh), slice_cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.flexsae_topk_bwd(ctypes.byref(sh), ptr(begin), ptr(mp), ptr(indices if pass_indices else None),
                              ptr(weight), ptr(vals), ptr(resid),
                              ptr(g), ptr(dW), DT[dw_dtype], ptr(dv), ptr(db), ptr(ws), nbytes, flags, stream())
    return rc, dW, dv, db


def cast_from_f32(src, dtype):
    lib = _lib.load()
    dst = torch.empty(src.shape, dtype=dtype, device=src.device)
    rc = lib.flexsae_cast_from_f32(ptr(dst), DT[dtype], ptr(src), src.numel(), stream())
    return rc, dst
