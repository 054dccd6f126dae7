"""The five benchmark configurations at their full sizes.

Configurations 1-4 are compared element by element with the CPU oracle (double accumulation).
Configuration 5 is too large for that in a test's time budget, so it is checked (and 4 in
addition) through properties that do not depend on size:
  * parity with the oracle on a row subset, at the full F and D (so all 64-bit addressing of
    the weight matrix is exercised), the oracle working on the compacted set of touched rows;
  * additivity over the batch: loss and gradients of the whole batch equal the B-weighted
    combination of the results on disjoint row blocks;
  * conservation: sum_f <W[f], dW[f]> == sum_{b,k} vals * dvals;
  * rows of dW belonging to latents that no pair selects are exactly zero.
Tolerances: fp32 1e-5 (loss) / 1e-4 (gradients); bf16 1e-2; written next to each check.
"""
import numpy as np
import pytest
import torch

import flexsae_amd as flex
import oracle
from helpers import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
FUSED = {"hier": flex.triton_hierarchical_sae_loss, "topk": flex.triton_topk_sae_loss}
MODES = {"hier": oracle.HIER, "topk": oracle.TOPK}


def _gen(B, K, F, D, dtype, dist, w_std=1.0, seed=1234):
    """Inputs generated on the GPU (fast for the big shapes), indices/vals/weight/bias/target."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    if dist == "randint":
        idx = torch.randint(0, F, (B, K), generator=g, device=DEV)
    else:
        idx = torch.empty(B, K, dtype=torch.long, device=DEV)
        step = max(1, (1 << 26) // F)
        if dist == "zipf":
            logp = -1.1 * torch.log(torch.arange(1, F + 1, dtype=torch.float32, device=DEV))
            perm = torch.randperm(F, generator=g, device=DEV)
        for b0 in range(0, B, step):
            n = min(step, B - b0)
            u = torch.rand(n, F, generator=g, device=DEV)
            if dist == "zipf":
                key = logp - torch.log(-torch.log(u.clamp_(1e-30, 1 - 1e-7)))
                idx[b0:b0 + n] = perm[key.topk(K, dim=1).indices]
            else:
                idx[b0:b0 + n] = u.topk(K, dim=1).indices
    vals = torch.randn(B, K, generator=g, device=DEV).abs()
    if dist == "zipf":
        vals = vals.sort(dim=1, descending=True).values
    W = torch.empty(F, D, dtype=dtype, device=DEV)
    rows = max(1, (1 << 27) // D)
    for f0 in range(0, F, rows):
        n = min(rows, F - f0)
        W[f0:f0 + n] = (torch.randn(n, D, generator=g, device=DEV) * w_std).to(dtype)
    bias = torch.randn(D, generator=g, device=DEV).to(dtype)
    target = torch.randn(B, D, generator=g, device=DEV).to(dtype)
    return idx, W, vals.to(dtype), bias, target


def _run(mode, idx, W, v, b, t, grad_out=1.0):
    Wp, vp, bp = (x.detach().clone().requires_grad_() for x in (W, v, b))
    loss = FUSED[mode](idx, Wp, vp, bp, t)
    loss.backward(torch.tensor(grad_out, device=DEV))
    torch.cuda.synchronize()
    return loss.detach(), Wp.grad, vp.grad, bp.grad


def _elementwise(name, got, ref, tol):
    """The parity bar for one gradient tensor: ||got - ref|| <= tol ||ref|| and, element by element,
    |got - ref| <= tol |ref| + tol max|ref| (float64, in row blocks to bound the memory)."""
    got2, ref2 = got.reshape(-1, got.shape[-1]), ref.reshape(-1, ref.shape[-1])
    ref_max = float(ref2.abs().max())
    num = den = 0.0
    worst = -1.0
    blk = max(1, (1 << 24) // ref2.shape[1])
    for r0 in range(0, ref2.shape[0], blk):
        g, r = got2[r0:r0 + blk].double(), ref2[r0:r0 + blk].double()
        diff = (g - r).abs()
        num += float((diff ** 2).sum())
        den += float((r ** 2).sum())
        worst = max(worst, float((diff - tol * r.abs()).max()) - tol * ref_max)
    assert num ** 0.5 <= tol * den ** 0.5, f"{name}: rel err {(num / den) ** 0.5:.3e} > {tol}"
    assert worst <= 0, f"{name}: an element misses rtol={tol}, atol={tol}*max|ref| by {worst:.3e}"


def _full_compare(mode, args, dtype, grad_out, tol_loss, tol_grad):
    idx, W, v, b, t = args
    loss, dW, dv, db = _run(mode, *args, grad_out=grad_out)
    cpu = [x.cpu() for x in args]
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], *cpu, grad_out=grad_out, dw_float32=True)
    assert abs(loss.item() - L) <= tol_loss * abs(L), (loss.item(), L)
    _elementwise("dvals", dv.cpu(), torch.from_numpy(rv), tol_grad)
    _elementwise("dbias", db.cpu(), torch.from_numpy(rb), tol_grad)
    # dW on the GPU (the matrices are large): normwise and element by element
    _elementwise("dW", dW, torch.from_numpy(rW).to(DEV), tol_grad)
    touched = torch.zeros(W.shape[0], dtype=torch.bool, device=DEV)
    touched[idx.flatten()] = True
    assert torch.count_nonzero(dW[~touched]) == 0


@pytest.mark.parametrize("mode", ["topk", "hier"])
def test_config1_fp32_small(mode):
    print("[case] config1", mode, flush=True)
    args = _gen(64, 32, 4096, 256, torch.float32, "randint")
    _full_compare(mode, args, torch.float32, 1.0, 1e-5, 1e-4)


@pytest.mark.parametrize("mode,K", [("hier", 128), ("topk", 128), ("hier", 32), ("hier", 64), ("topk", 32),
                                    ("topk", 64)])
def test_config2_bf16(mode, K):
    print("[case] config2", mode, K, flush=True)
    args = _gen(4096, K, 65536, 2304, torch.bfloat16, "unique")
    assert all(len(set(r.tolist())) == K for r in args[0][:8].cpu())  # per-row unique
    _full_compare(mode, args, torch.bfloat16, 0.5, 1e-2, 1e-2)


def test_config3_fp32_duplicates():
    print("[case] config3", flush=True)
    args = _gen(2048, 256, 131072, 1024, torch.float32, "randint")
    _full_compare("hier", args, torch.float32, 1.0, 1e-5, 1e-4)


def _subset_parity(mode, args, rows, tol_loss, tol_grad):
    """`rows`: a slice of the batch rows (an int n means the first n)."""
    idx, W, v, b, t = args
    sl = slice(0, rows) if isinstance(rows, int) else rows
    sub = (idx[sl].contiguous(), W, v[sl].contiguous(), b, t[sl].contiguous())
    loss, dW, dv, db = _run(mode, *sub)
    # oracle on the compacted problem: only the rows of W that the subset touches
    uniq, inv = torch.unique(sub[0], return_inverse=True)
    Wc = W[uniq].float().cpu()
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], inv.cpu(), Wc, sub[2].cpu(), b.cpu(), sub[4].cpu(),
                                      dw_float32=True)
    assert abs(loss.item() - L) <= tol_loss * abs(L), (loss.item(), L)
    _elementwise("dvals", dv.cpu(), torch.from_numpy(rv), tol_grad)
    _elementwise("dbias", db.cpu(), torch.from_numpy(rb), tol_grad)
    _elementwise("dW", dW[uniq].cpu(), torch.from_numpy(rW), tol_grad)
    mask = torch.ones(W.shape[0], dtype=torch.bool, device=DEV)
    mask[uniq] = False
    assert torch.count_nonzero(dW[mask]) == 0


def _additivity_and_conservation(mode, args, n_blocks, tol):
    idx, W, v, b, t = args
    B = idx.shape[0]
    loss, dW, dv, db = _run(mode, *args)
    acc_loss = 0.0
    acc_dW = torch.zeros(W.shape, dtype=torch.float32, device=DEV)
    acc_db = torch.zeros(b.shape, dtype=torch.float32, device=DEV)
    step = B // n_blocks
    for b0 in range(0, B, step):
        sl = slice(b0, b0 + step)
        l_, dW_, dv_, db_ = _run(mode, idx[sl].contiguous(), W, v[sl].contiguous(), b, t[sl].contiguous())
        w8 = step / B
        acc_loss += l_.item() * w8
        acc_dW += dW_.float() * w8
        acc_db += db_.float() * w8
        # dvals of a row only depend on that row, up to the 1/B normalisation
        assert rel_err((dv_.float() * w8).cpu(), dv[sl].float().cpu()) <= tol
        del dW_
    assert abs(loss.item() - acc_loss) <= tol * abs(acc_loss)
    num = (dW.float() - acc_dW).double().norm().item()
    den = acc_dW.double().norm().item()
    assert num / den <= tol, f"additivity of dW: {num / den:.3e}"
    assert rel_err(db.float().cpu(), acc_db.cpu()) <= tol
    lhs = 0.0
    blk = max(1, W.shape[0] // 16)
    for f0 in range(0, W.shape[0], blk):  # in row blocks: the full product would be tens of GB
        lhs += (W[f0:f0 + blk].double() * dW[f0:f0 + blk].double()).sum().item()
    rhs = (v.double() * dv.double()).sum().item()
    assert abs(lhs - rhs) <= tol * abs(rhs), (lhs, rhs)


def test_config4_bf16_zipf():
    print("[case] config4", flush=True)
    args = _gen(8192, 64, 262144, 4096, torch.bfloat16, "zipf", w_std=0.02)
    counts = torch.bincount(args[0].flatten(), minlength=262144)
    assert counts.max().item() > 4096  # the hottest latent is in most rows
    # every gradient of the full batch against the oracle, element by element: the latents with
    # thousands of pairs only exist at the full size
    _full_compare("hier", args, torch.bfloat16, 0.5, 1e-2, 1e-2)
    _additivity_and_conservation("hier", args, 4, 1e-2)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_config5_bf16_large(mode):
    print("[case] config5", mode, flush=True)
    args = _gen(16384, 128, 524288, 8192, torch.bfloat16, "unique", w_std=0.02)
    _subset_parity(mode, args, 1024, 1e-2, 1e-2)
    _subset_parity(mode, args, slice(16384 - 1024, 16384), 1e-2, 1e-2)  # the far end of every per-pair array
    _additivity_and_conservation(mode, args, 2, 1e-2)
    del args
    torch.cuda.empty_cache()
