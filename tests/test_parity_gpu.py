"""GPU parity tests: HIP kernels (through the C-ABI and through the torch ops) vs the CPU oracle.

Tolerances (normwise relative error, ||got-ref|| / ||ref||):
  fp32 : 1e-5 on the loss, 1e-4 on dvals / dW / dbias
  bf16 : 1e-2 on everything;  fp16 : 1e-3
and, on the reference's own shape x dtype matrix, also torch.testing.assert_close with the
reference's per-dtype atol/rtol (reference tests/test_setup.py:35-39).  Integer outputs (the
latent-major pair list) and gather addressing are compared bit for bit.
"""
import numpy as np
import pytest
import torch

import abi
import flexsae_amd as flex
from flexsae_amd import _lib
import oracle
from helpers import DTYPE_TO_TOLS, PARAMS, REL_TOL, make_inputs, rel_err

pytestmark = pytest.mark.gpu

DEV = "cuda"
MODES = {"hier": oracle.HIER, "topk": oracle.TOPK}
FUSED = {"hier": flex.triton_hierarchical_sae_loss, "topk": flex.triton_topk_sae_loss}


def _to_dev(args):
    return [a.to(DEV) for a in args]


def _announce(*what):
    print("[case]", *what, flush=True)


STAGE_ALL = 1 << 40  # a stage budget that holds the contributions of every test shape


def _run_op(mode, args_cpu, grad_out):
    idx, W, v, b, t = _to_dev(args_cpu)
    W.requires_grad_()
    v.requires_grad_()
    b.requires_grad_()
    loss = FUSED[mode](idx, W, v, b, t)
    loss.backward(torch.tensor(grad_out, device=DEV, dtype=torch.float32))
    torch.cuda.synchronize()
    assert idx.grad is None and t.grad is None
    return loss, W.grad, v.grad, b.grad


def check_gradient(name, got, ref, dtype, tol):
    """The parity bar for one gradient tensor against the oracle's float64 result:
    normwise ||got - ref|| <= tol * ||ref||, and element by element
    |got - ref| <= tol * |ref| + tol * max|ref|.
    fp32 and bf16 leaves get exactly that.  fp16 leaves get, on top, what rounding the exact
    gradient to fp16 costs by itself: gradients of magnitude 2/(B*K*D) are subnormal in fp16
    (spacing 6e-8), so their rounding error alone can exceed any relative tolerance."""
    ref_t = torch.as_tensor(ref, dtype=torch.float64)
    got_t = got.detach().double().cpu()
    err = rel_err(got_t, ref_t)
    quant_rel, quant_abs = 0.0, 0.0
    if dtype == torch.float16:
        rounded = ref_t.to(dtype).double()
        quant_rel = 1.5 * rel_err(rounded, ref_t)
        quant_abs = 1.5 * float((rounded - ref_t).abs().max())
    assert err <= tol + quant_rel, f"{name}: rel err {err:.3e} > {tol} (+ {quant_rel:.3e})"
    bound = tol * ref_t.abs() + tol * float(ref_t.abs().max()) + quant_abs
    worst = float(((got_t - ref_t).abs() - bound).max())
    assert worst <= 0, f"{name}: an element misses rtol={tol}, atol={tol}*max|ref| by {worst:.3e}"


def _check_against_oracle(mode, args_cpu, dtype, grad_out, got, ref_tols=True):
    loss, dW, dv, db = got
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], *args_cpu, grad_out=grad_out)
    tol_loss, tol_grad = REL_TOL[dtype]
    assert loss.dtype == torch.float32 and loss.dim() == 0
    assert abs(loss.item() - L) <= tol_loss * abs(L), (loss.item(), L)
    assert dW.dtype == dtype and dv.dtype == dtype and db.dtype == dtype
    for name, g, r in (("dW", dW, rW), ("dvals", dv, rv), ("dbias", db, rb)):
        check_gradient(name, g, r, dtype, tol_grad)
    if ref_tols:
        tols = DTYPE_TO_TOLS[dtype]
        torch.testing.assert_close(loss.cpu(), torch.tensor(L, dtype=torch.float32), **tols)
        for g, r in ((dW, rW), (dv, rv), (db, rb)):
            torch.testing.assert_close(g.cpu(), torch.from_numpy(r).to(dtype), **tols)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("B,K,F,D", PARAMS)
@pytest.mark.parametrize("mode", ["hier", "hier_staged", "topk"])
def test_reference_matrix(mode, B, K, F, D, dtype):
    """The reference's 26 shapes x 3 dtypes x 2 losses, with a random scalar upstream gradient
    (reference tests/test_all_kernels.py:20-66).  The hierarchical loss runs in both memory modes:
    flat (the default: training step slice by slice) and with all contributions staged."""
    _announce("matrix", mode, B, K, F, D, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype)
    grad_out = float(torch.randn((), generator=torch.Generator().manual_seed(B * K + D)))
    flex.set_hier_stage_bytes(STAGE_ALL if mode == "hier_staged" else None)
    try:
        got = _run_op(mode.split("_")[0], args, grad_out)
    finally:
        flex.set_hier_stage_bytes(None)
    _check_against_oracle(mode.split("_")[0], args, dtype, grad_out, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("B,K,F,D", PARAMS[::3])
def test_reference_matrix_without_fused_training(B, K, F, D, dtype):
    """The hierarchical loss takes the fused forward+backward pass by default when gradients are
    required; this runs every third shape through the separate forward / backward kernels."""
    _announce("matrix unfused", B, K, F, D, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype)
    flex.set_fused_training(False)
    try:
        got = _run_op("hier", args, -0.6)
    finally:
        flex.set_fused_training(True)
    _check_against_oracle("hier", args, dtype, -0.6, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape", [(48, 32, 200, 768), (7, 5, 300, 260), (33, 128, 64, 2304), (16, 64, 9, 132),
                                   (5, 100, 40, 512), (64, 16, 1000, 4), (9, 256, 700, 320), (6, 130, 50, 192),
                                   (12, 200, 3000, 72), (40, 16, 200, 512), (50, 8, 333, 640)])
def test_training_step_entry_point(shape, dtype):
    """flexsae_hier_fwd_bwd through the C-ABI: loss and unit-gradient gradients in one pass, for
    K that are and are not powers of two, up to 256 (the kernel variants with and without row
    pieces in the LDS), D that are not whole tiles, hot latents (F tiny), and between one and
    four pairs per latent on average (with at most two the reduction serves four latents per group of lanes)."""
    B, K, F, D = shape
    _announce("train abi", shape, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=41)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, dW, dv, db = abi.hier_train(idx, W, v, b, t)
    torch.cuda.synchronize()
    assert rc == 0
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *args, grad_out=1.0)
    tol_loss, _ = REL_TOL[dtype]
    assert abs(loss.item() - L) <= tol_loss * abs(L)
    assert rel_err(dW.cpu(), rW) < (4e-3 if dtype == torch.bfloat16 else 1e-4)
    assert rel_err(dv.cpu(), rv) < 1e-4 and rel_err(db.cpu(), rb) < 1e-4
    # bit-identical dW for any slice width, and equal to the two-kernel path's
    rc2, _, dW2, _, _ = abi.hier_train(idx, W, v, b, t, slice_cols=1 << 20)
    assert rc2 == 0 and torch.equal(dW, dW2)
    rc3, loss3, resid = abi.forward("hier", idx, W, v, b, t)
    rc4, dW4, dv4, db4 = abi.hier_backward(idx, W, v, resid, 1.0)
    assert rc3 == rc4 == 0
    assert abs(loss.item() - loss3.item()) <= 2e-6 * abs(L)
    assert rel_err(dW.cpu(), dW4.cpu()) < (4e-3 if dtype == torch.bfloat16 else 2e-5)
    assert rel_err(dv.cpu(), dv4.cpu()) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape", [(48, 32, 200, 768), (33, 128, 64, 2304), (9, 256, 700, 320), (64, 16, 1000, 8),
                                   (40, 16, 200, 512), (50, 8, 333, 640), (16, 64, 9, 136)])
def test_sgd_step_entry_point(shape, dtype):
    """flexsae_hier_sgd_step through the C-ABI: W_new = W - step * dW of the oracle on the touched rows
    (one rounding to the weight's dtype), untouched rows bit-identical to before, loss / dvals / dbias
    bit-identical to flexsae_hier_fwd_bwd's (they come from the weights as they were on entry), for any
    slice width."""
    B, K, F, D = shape
    _announce("sgd step abi", shape, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=43)
    idx, W, v, b, t = _to_dev(args)
    step = 0.37
    rc0, loss0, dW0, dv0, db0 = abi.hier_train(idx, W, v, b, t)
    assert rc0 == 0
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *args, grad_out=1.0)
    touched = torch.zeros(F, dtype=torch.bool)
    touched[args[0].flatten()] = True
    for cols in (0, 1 << 20):
        Wn = W.clone()
        rc, loss, dv, db = abi.hier_sgd_step(idx, Wn, v, b, t, step, slice_cols=cols)
        torch.cuda.synchronize()
        assert rc == 0, _lib.status_string(rc)
        assert torch.equal(loss, loss0) and torch.equal(dv, dv0) and torch.equal(db, db0)
        Wn = Wn.cpu()
        assert torch.equal(Wn[~touched], args[1][~touched])
        # the kernel's own fp32 gradient, rounded once: identical bits
        expect = (W.float() - step * dW0).to(dtype).cpu()
        if dtype == torch.float32:  # w - step*g may be contracted into one fused multiply-add
            assert rel_err(Wn[touched], expect[touched]) < 1e-6
        else:
            assert (Wn[touched].float() - expect[touched].float()).abs().max() <= \
                torch.finfo(dtype).eps * expect[touched].float().abs().max()
        # and against the oracle: the update itself, not the updated weights (which it barely moves)
        upd = (args[1].float()[touched] - Wn[touched].float()) / step
        ref = torch.from_numpy(rW).float()[touched]
        # rounding W_new to the weight's dtype quantises the recovered update at eps*|W|/step
        quant = torch.finfo(dtype).eps * args[1].float().abs().max() / step
        tol = 1e-4 if dtype == torch.float32 else 1e-2
        assert (upd - ref).abs().max() <= tol * ref.abs().max() + quant


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("D", [384, 256, 72])
def test_sparse_latents_take_the_row_count_list(D, dtype):
    """B*K <= 2F with skewed indices: most latents have no pair, the others between one and several
    hundred.  The reduction then works from the list of latents ordered by row count and the rows of
    latents without pairs are zeroed in one pass: every row of dW (handed over full of NaN) must come
    out written, exactly zero where the latent has no pair, equal to the oracle elsewhere, for slices
    of one, three and all column pieces; the in-place SGD variant must leave the rows without pairs
    alone and move the others by the same gradient."""
    B, K, F = 768, 16, 8192
    _announce("sparse class list", (B, K, F, D), dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=101, zipf_s=1.1, sort_vals=True, w_std=0.05)
    counts = torch.bincount(args[0].flatten(), minlength=F)
    assert B * K <= 2 * F and (counts == 0).sum() > F // 2 and counts.max() > 64
    assert len(set(counts[(counts > 0) & (counts <= 64)].tolist())) >= 12  # many row-count classes in use
    idx, W, v, b, t = _to_dev(args)
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *args, grad_out=1.0)
    rW = torch.from_numpy(rW)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-4
    first = None
    for cols in (0, 3 * 128, 1 << 20):
        rc, loss, dW, dv, db = abi.hier_train(idx, W, v, b, t, slice_cols=cols, dw_dtype=dtype)
        torch.cuda.synchronize()
        assert rc == 0, _lib.status_string(rc)
        dWc = dW.float().cpu()
        assert not torch.isnan(dWc).any()
        assert (dWc[counts == 0] == 0).all()
        check_gradient("dW", dWc, rW, dtype, tol)
        assert rel_err(dv.cpu(), rv) < tol and rel_err(db.cpu(), rb) < tol
        if first is None:
            first = dW
        assert torch.equal(dW, first)  # same bits for any slice width
    step = 0.25
    Wn = W.clone()
    rc, loss2, dv2, db2 = abi.hier_sgd_step(idx, Wn, v, b, t, step)
    torch.cuda.synchronize()
    assert rc == 0, _lib.status_string(rc)
    assert torch.equal(Wn[(counts == 0).to(Wn.device)], W[(counts == 0).to(W.device)])
    upd = ((W.float() - Wn.float()) / step).cpu()
    quant = torch.finfo(dtype).eps * args[1].float().abs().max() / step
    assert (upd - rW.float()).abs().max() <= tol * rW.abs().max() + quant


def test_sgd_step_through_the_package():
    """hierarchical_sae_sgd_step: one fused call equals loss.backward() + plain SGD on the decoder
    weight; dvals and dbias are those of the autograd path; repeated steps lower the loss."""
    args = make_inputs(64, 32, 500, 512, dtype=torch.float32, seed=44)
    idx, W, v, b, t = _to_dev(args)
    lr = 0.05
    Wa = W.clone().requires_grad_()
    va, ba = v.clone().requires_grad_(), b.clone().requires_grad_()
    loss_a = flex.triton_hierarchical_sae_loss(idx, Wa, va, ba, t)
    loss_a.backward()
    W_sgd = (Wa.detach() - lr * Wa.grad)
    Wf = W.clone().requires_grad_()   # a leaf that requires grad: updated in place without autograd
    loss_f, dv, db = flex.hierarchical_sae_sgd_step(idx, Wf, v, b, t, lr)
    torch.cuda.synchronize()
    assert torch.equal(loss_f, loss_a.detach())
    assert rel_err(Wf.detach().cpu(), W_sgd.cpu()) < 1e-6
    assert torch.equal(dv, va.grad) and torch.equal(db, ba.grad)
    losses = [loss_f.item()]
    for _ in range(5):
        l, _, _ = flex.hierarchical_sae_sgd_step(idx, Wf, v, b, t, 20.0)
        losses.append(l.item())
    assert all(x > y for x, y in zip(losses, losses[1:])), losses
    # an upstream gradient scales the step
    W2 = W.clone()
    flex.hierarchical_sae_sgd_step(idx, W2, v, b, t, lr, grad_out=torch.tensor(2.0, device=DEV))
    assert rel_err(W2.cpu(), (W - 2 * lr * Wa.grad).cpu()) < 1e-6
    with pytest.raises(ValueError):
        flex.hierarchical_sae_sgd_step(idx, W.t().contiguous().t(), v, b, t, lr)


def test_sgd_step_unsupported_shapes():
    idx, W, v, b, t = _to_dev(make_inputs(8, 8, 32, 12, dtype=torch.bfloat16, seed=3))  # D % 8 != 0 with 16-bit weights
    rc, *_ = abi.hier_sgd_step(idx, W.clone(), v, b, t, 0.1)
    assert rc == -2
    idx, W, v, b, t = _to_dev(make_inputs(8, 8, 32, 12, seed=3))  # fp32: a multiple of 4 is enough
    rc, *_ = abi.hier_sgd_step(idx, W.clone(), v, b, t, 0.1)
    assert rc == 0


def test_training_step_unsupported_shapes_and_scale():
    idx, W, v, b, t = _to_dev(make_inputs(8, 8, 32, 6, seed=3))  # D % 4 != 0
    rc, *_ = abi.hier_train(idx, W, v, b, t)
    assert rc == -2
    idx, W, v, b, t = _to_dev(make_inputs(4, 260, 32, 64, dtype=torch.bfloat16, seed=3))  # K > 256
    rc, *_ = abi.hier_train(idx, W, v, b, t)
    assert rc == -2
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        x = torch.randn(1003, device=DEV).to(dt)
        rc, y = abi.scale(x, -2.5)
        assert rc == 0 and torch.equal(y, (x.float() * -2.5).to(dt))
        for g in (1.0, 0.75):  # in place; by one the kernel leaves everything as it is
            z = x.clone()
            rc, z2 = abi.scale(z, g, in_place=True)
            assert rc == 0 and z2 is z and torch.equal(z, (x.float() * g).to(dt))


def test_training_step_without_dw():
    """FLEXSAE_BWD_NO_DW: loss, dvals and dbias as usual, for any workspace width; dW is not touched."""
    args = make_inputs(40, 32, 300, 1024, dtype=torch.bfloat16, seed=19)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, dW, dv, db = abi.hier_train(idx, W, v, b, t, dw_dtype=torch.bfloat16)
    assert rc == 0
    for cols in (0, 256, 1 << 20):
        rc2, loss2, dW2, dv2, db2 = abi.hier_train(idx, W, v, b, t, slice_cols=cols, dw_dtype=torch.bfloat16, flags=32)
        torch.cuda.synchronize()
        assert rc2 == 0 and torch.equal(loss, loss2) and torch.equal(dv, dv2) and torch.equal(db, db2)
        assert torch.isnan(dW2.float()).all()
    # measurement aid: without the epilogue kernels nothing but the contributions is written
    rc3, loss3, dW3, dv3, db3 = abi.hier_train(idx, W, v, b, t, dw_dtype=torch.bfloat16, flags=32 | 64)
    torch.cuda.synchronize()
    assert rc3 == 0 and torch.isnan(loss3).all() and torch.isnan(dv3).all() and torch.isnan(dW3.float()).all()


@pytest.mark.parametrize("stage", [STAGE_ALL, None], ids=["staged", "sliced"])
def test_fused_training_backward_twice_and_no_grad(stage):
    """retain_graph + two backward calls accumulate correctly; no_grad / non-leaf-free inputs take
    the forward-only kernel."""
    args = make_inputs(32, 16, 100, 512, dtype=torch.bfloat16, seed=8)
    idx, W, v, b, t = _to_dev(args)
    W.requires_grad_()
    flex.set_hier_stage_bytes(stage)
    try:
        loss = flex.triton_hierarchical_sae_loss(idx, W, v, b, t)
        loss.backward(torch.tensor(2.0, device=DEV), retain_graph=True)
        g1 = W.grad.clone()
        loss.backward(torch.tensor(-0.5, device=DEV))
    finally:
        flex.set_hier_stage_bytes(None)
    L, rW, _, _ = oracle.loss_grads(oracle.HIER, *args, grad_out=1.5)
    assert rel_err(W.grad.float().cpu(), rW) < 2e-2
    assert rel_err(g1.float().cpu(), rW * (2.0 / 1.5)) < 1e-2
    with torch.no_grad():
        l2 = flex.triton_hierarchical_sae_loss(idx, W, v, b, t)
    assert not l2.requires_grad and abs(l2.item() - loss.item()) <= 2e-6 * abs(L)


@pytest.mark.parametrize("mode", ["hier", "topk"])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (3, 5, 7, 9), (5, 3, 11, 70), (2, 65, 40, 130),
                                   (7, 130, 300, 200), (4, 24, 50, 1000), (33, 12, 17, 2304), (3, 300, 900, 136),
                                   (2, 512, 4096, 64)])
def test_odd_shapes_fp32(mode, shape):
    """Sizes the reference's static asserts reject: K not a power of two, K > 64 with a ragged
    last group, D not a multiple of 64 (nor of the vector width), B not a multiple of 16; rows of
    more than 256 steps (forward + sliced backward instead of the training-step kernel)."""
    B, K, F, D = shape
    _announce("odd", mode, shape)
    args = make_inputs(B, K, F, D, seed=B + K + F + D)
    got = _run_op(mode, args, -1.25)
    _check_against_oracle(mode, args, torch.float32, -1.25, got, ref_tols=False)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_mixed_dtypes(mode):
    """weight/vals/bias/target each in a different dtype (the reference upcasts each load on its
    own: hierarchical_kernels.py:49-64, topk_kernels.py:38)."""
    _announce("mixed", mode)
    idx, W, v, b, t = make_inputs(24, 16, 90, 384, seed=21)
    args = (idx, W.to(torch.bfloat16), v.to(torch.float16), b.to(torch.float32), t.to(torch.float16))
    loss, dW, dv, db = _run_op(mode, args, 0.5)
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], *args, grad_out=0.5)
    assert abs(loss.item() - L) <= 1e-5 * abs(L)
    assert (dW.dtype, dv.dtype, db.dtype) == (torch.bfloat16, torch.float16, torch.float32)
    assert rel_err(dW.float().cpu(), rW) < 1e-2
    assert rel_err(dv.float().cpu(), rv) < 1e-3
    assert rel_err(db.cpu(), rb) < 1e-4


@pytest.mark.parametrize("mode", ["hier", "topk"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_gather_addressing_is_exact(mode, dtype):
    """Identity-style weight: W[f,d] holds an integer code of (f,d), vals = 1, bias = target = 0,
    so resid[b,d] is an exact integer sum that reveals precisely which addresses were read."""
    B, K, F = 37, 4, 1000
    D = 512 if dtype == torch.float32 else 64
    _announce("addressing", mode, dtype)
    g = torch.Generator().manual_seed(3)
    idx = torch.randint(0, F, (B, K), generator=g)
    if dtype == torch.float32:
        W = (torch.arange(F).unsqueeze(1) * D + torch.arange(D)).float()  # < 2^24, exact
    else:
        W = ((torch.arange(F).unsqueeze(1) * 7 + torch.arange(D) * 3) % 64).float()  # exact in bf16
    v = torch.ones(B, K)
    args = [idx, W.to(dtype), v.to(dtype), torch.zeros(D, dtype=dtype), torch.zeros(B, D, dtype=dtype)]
    rc, loss, resid = abi.forward(mode, *_to_dev(args))
    assert rc == 0
    expect = W[idx].sum(dim=1)  # exact in fp32: integer sums below 2^24
    assert torch.equal(resid.cpu(), expect)


@pytest.mark.parametrize("shape", [(4, 8, 16), (37, 16, 5), (64, 32, 4096), (192, 256, 512), (300, 70, 3),
                                   (128, 64, 100000), (2048, 33, 1), (4096, 128, 65536), (1000, 100, 700),
                                   (64, 16, (1 << 25)), (64, 16, (1 << 25) + 7), (3000, 40, 9000, "skew")])
def test_pair_list_bit_exact(shape):
    """begin/map equal the stable counting sort (oracle = numpy argsort(kind='stable')).  The shapes cover
    one bucket and many, buckets sorted in the LDS and buckets too large for it, latents with more than 64
    pairs, the largest bucket count, and (F above 2^25) the construction with memory atomics."""
    B, K, F = shape[:3]
    _announce("csr", shape)
    g = torch.Generator().manual_seed(B + K + F)
    if len(shape) > 3:  # a few hot latents next to a long uniform tail
        hot = torch.randint(0, 12, (B, K), generator=g) * 613 % F
        idx = torch.where(torch.rand(B, K, generator=g) < 0.4, hot, torch.randint(0, F, (B, K), generator=g))
    else:
        idx = torch.randint(0, F, (B, K), generator=g)
    rbegin, rmap = oracle.csr(idx, F)
    for _ in range(2):  # twice: the result may not depend on how the atomics were served
        rc, begin, mp = abi.csr_build(idx.to(DEV), F)
        torch.cuda.synchronize()
        assert rc == 0
        np.testing.assert_array_equal(abi.widen_u32(begin).cpu().numpy(), rbegin.astype(np.int64))
        np.testing.assert_array_equal(abi.widen_u32(mp).cpu().numpy(), rmap.astype(np.int64))


@pytest.mark.parametrize("mode", ["hier", "topk"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_c_abi_direct(mode, dtype):
    """Forward and backward entry points called with raw pointers; outputs start as NaN so a
    missing zero-fill or an unwritten element shows."""
    B, K, F, D = 48, 32, 200, 768
    _announce("abi", mode, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=17)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward(mode, idx, W, v, b, t)
    assert rc == 0
    if mode == "hier":
        rc, dW, dv, db = abi.hier_backward(idx, W, v, resid, 0.7)
        rc2, dW2, dv2, db2 = abi.hier_backward_atomic(idx, W, v, resid, 0.7)
        assert rc2 == 0
        tol = 1e-4 if dtype == torch.float32 else 4e-3  # bf16 weights: contributions pass through bf16
        assert rel_err(dW.cpu(), dW2.cpu()) < tol
        assert rel_err(dv.cpu(), dv2.cpu()) < 1e-5 and rel_err(db.cpu(), db2.cpu()) < 1e-5
    else:
        rc, dW, dv, db = abi.topk_backward(idx, W, v, resid, 0.7, dw_dtype=torch.float32)
    assert rc == 0
    torch.cuda.synchronize()
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], *args, grad_out=0.7)
    tol_loss, _ = REL_TOL[dtype]
    assert abs(loss.item() - L) <= tol_loss * abs(L)
    # outputs here are fp32 whatever the input dtype, so the fp32 bar applies to the arithmetic,
    # except that for bf16 weights the two-phase hierarchical backward stores bf16 contributions
    # and the TopK backward gathers a bf16 copy of the residual (as the reference's does)
    assert rel_err(dW.cpu(), rW) < (4e-3 if dtype == torch.bfloat16 else 1e-4)
    assert rel_err(dv.cpu(), rv) < (4e-3 if (mode == "topk" and dtype == torch.bfloat16) else 1e-4)
    assert rel_err(db.cpu(), rb) < 1e-4
    # resid is r_{K-1} - target
    rW0 = W.float().cpu()[idx.cpu()] * v.float().cpu().unsqueeze(-1)
    expect = b.float().cpu() + rW0.sum(1) - t.float().cpu()
    assert rel_err(resid.cpu(), expect) < 1e-5
    # untouched latents: exactly zero rows
    untouched = np.setdiff1d(np.arange(F), idx.cpu().numpy().ravel())
    if untouched.size:
        assert torch.count_nonzero(dW[torch.from_numpy(untouched).to(DEV)]) == 0


def test_hier_atomic_prezeroed_flag_and_cast():
    args = make_inputs(16, 16, 64, 512, dtype=torch.bfloat16, seed=5)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward("hier", idx, W, v, b, t)
    rc1, dW1, dv1, db1 = abi.hier_backward_atomic(idx, W, v, resid, 1.0)
    rc2, dW2, dv2, db2 = abi.hier_backward_atomic(idx, W, v, resid, 1.0, prezeroed=True)
    assert rc == rc1 == rc2 == 0
    assert rel_err(dW2.cpu(), dW1.cpu()) < 1e-6 and rel_err(db2.cpu(), db1.cpu()) < 1e-6
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        rc, out = abi.cast_from_f32(dW1, dt)
        assert rc == 0
        assert torch.equal(out, dW1.to(dt))  # same round-to-nearest-even as torch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(64, 32, 224, 1024), (33, 12, 17, 2304), (96, 130, 9, 200), (256, 64, 3, 70)])
def test_hier_slice_width_does_not_change_the_result(shape, dtype):
    """The slice width only sets how many passes are made: dW must come out bit-identical for
    any workspace size, also with long groups (F tiny => hot latents cut into chunks) and
    with D that is not a whole number of tiles."""
    B, K, F, D = shape
    _announce("slices", shape, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=31)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward("hier", idx, W, v, b, t)
    assert rc == 0
    outs = []
    for cols in (0, 512, 1 << 20):
        rc, dW, dv, db = abi.hier_backward(idx, W, v, resid, -0.3, slice_cols=cols)
        assert rc == 0
        outs.append((dW, dv, db))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[1][0], outs[2][0])
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *args, grad_out=-0.3)
    assert rel_err(outs[0][0].cpu(), rW) < (4e-3 if dtype == torch.bfloat16 else 1e-4)
    for _, dv, db in outs:
        assert rel_err(dv.cpu(), rv) < 1e-4 and rel_err(db.cpu(), rb) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(64, 32, 224, 1024), (33, 12, 17, 2304), (96, 130, 9, 200), (256, 64, 3, 70)])
def test_topk_slice_width_does_not_change_the_result(shape, dtype):
    """Same for the TopK backward: hot latents (F tiny) go through 64-pair chunks whose partial
    sums live in a slice-wide workspace; any slice width must give bit-identical dW."""
    B, K, F, D = shape
    _announce("topk slices", shape, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=32)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward("topk", idx, W, v, b, t)
    assert rc == 0
    outs = []
    for cols in (0, 512, 1 << 20):
        rc, dW, dv, db = abi.topk_backward(idx, W, v, resid, 0.9, dw_dtype=torch.float32, slice_cols=cols)
        assert rc == 0
        outs.append((dW, dv, db))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[1][0], outs[2][0])
    assert torch.equal(outs[0][2], outs[1][2])  # dbias: fixed-order column sums
    L, rW, rv, rb = oracle.loss_grads(oracle.TOPK, *args, grad_out=0.9)
    tol = 4e-3 if dtype == torch.bfloat16 else 1e-4  # bf16 weights: bf16 copy of the residual
    assert rel_err(outs[0][0].cpu(), rW) < tol
    for _, dv, db in outs:
        assert rel_err(dv.cpu(), rv) < tol and rel_err(db.cpu(), rb) < 1e-4


@pytest.mark.parametrize("mode", ["hier", "topk"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_skewed_latents(mode, dtype):
    """Zipf-distributed per-row-unique indices with vals sorted descending (the shape of the
    skewed benchmark configuration, scaled down): a few latents appear in almost every row."""
    B, K, F, D = 512, 16, 4096, 512
    _announce("zipf", mode, dtype)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=77, zipf_s=1.1, sort_vals=True, w_std=0.02)
    counts = torch.bincount(args[0].flatten(), minlength=F)
    assert counts.max() > 300  # hot latents really are hot
    got = _run_op(mode, args, 1.0)
    _check_against_oracle(mode, args, dtype, 1.0, got, ref_tols=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_hier_gradients_are_reproducible_bit_for_bit(dtype):
    """dW (segment sums in list order), dvals (per-tile shares added in tile order) and dbias
    (fixed-order column sums) of both hierarchical entry points repeat exactly."""
    args = _to_dev(make_inputs(96, 32, 64, 1536, dtype=dtype, seed=9))  # F small: long groups, collisions
    idx, W, v, b, t = args
    _, _, resid = abi.forward("hier", *args)
    outs = [abi.hier_backward(idx, W, v, resid, 1.0)[1:] for _ in range(3)]
    for a, c in zip(outs[0], outs[1]):
        assert torch.equal(a, c)
    for a, c in zip(outs[1], outs[2]):
        assert torch.equal(a, c)
    outs = [abi.hier_train(idx, W, v, b, t)[1:] for _ in range(3)]
    for a, c in zip(outs[0], outs[1]):
        assert torch.equal(a, c)
    for a, c in zip(outs[1], outs[2]):
        assert torch.equal(a, c)


@pytest.mark.parametrize("mode", ["sliced", "segment", "atomic"])
def test_hier_backward_variants_through_the_op(mode):
    """What the public op runs when the stage budget is too small to keep a whole step's
    contributions: the training-step kernel slice by slice (1 MiB of scratch = several slices);
    with the fusion switched off, forward + sliced segment backward; with a scratch budget of 0,
    forward + the atomic fallback."""
    args = make_inputs(48, 32, 200, 768, dtype=torch.bfloat16, seed=13)
    flex.set_hier_scratch_bytes(0 if mode == "atomic" else 1 << 20)
    flex.set_hier_stage_bytes(1 << 20)
    flex.set_fused_training(mode != "segment")
    try:
        got = _run_op("hier", args, 1.5)
        if mode == "sliced":  # upstream gradient 1: bit-identical to the staged step
            one = _run_op("hier", args, 1.0)
            flex.set_hier_stage_bytes(STAGE_ALL)
            staged = _run_op("hier", args, 1.0)
            for a, c in zip(one, staged):
                assert torch.equal(a, c)
    finally:
        flex.set_hier_scratch_bytes(None)
        flex.set_hier_stage_bytes(None)
        flex.set_fused_training(True)
    _check_against_oracle("hier", args, torch.bfloat16, 1.5, got)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_loss_is_reproducible_bit_for_bit(mode):
    args = _to_dev(make_inputs(64, 32, 224, 1024, dtype=torch.bfloat16, seed=9))
    vals = {abi.forward(mode, *args)[1].item() for _ in range(5)}
    assert len(vals) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_topk_gradients_are_reproducible_bit_for_bit(dtype):
    args = _to_dev(make_inputs(96, 32, 64, 1536, dtype=dtype, seed=9))  # F small: long groups, collisions
    idx, W, v, b, t = args
    _, _, resid = abi.forward("topk", *args)
    outs = [abi.topk_backward(idx, W, v, resid, 1.0)[1:] for _ in range(3)]
    for a, c in zip(outs[0], outs[1]):
        assert torch.equal(a, c)
    for a, c in zip(outs[1], outs[2]):
        assert torch.equal(a, c)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_out_of_range_index_is_flagged_not_followed(mode):
    idx, W, v, b, t = make_inputs(8, 8, 32, 256, seed=1)
    idx[3, 2] = 32          # == F
    idx[5, 0] = -1
    args = _to_dev((idx, W, v, b, t))
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    rc, loss, resid = abi.forward(mode, *args, flag=flag)
    torch.cuda.synchronize()
    assert rc == 0 and flag.item() == 1
    # the offending pairs count as (latent 0, value 0): same result as zeroing them by hand
    idx2, v2 = idx.clone(), v.clone()
    idx2[3, 2] = idx2[5, 0] = 0
    v2[3, 2] = v2[5, 0] = 0
    L, *_ = oracle.loss_grads(MODES[mode], idx2, W, v2, b, t, want_grads=False)
    assert abs(loss.item() - L) <= 1e-5 * abs(L)
    # python layer: the check raises IndexError and clears the flag
    try:
        flex.check_index_flag()
    except IndexError:
        pass
    FUSED[mode](*args)
    with pytest.raises(IndexError):
        flex.check_index_flag()
    flex.check_index_flag()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("mode,path", [("hier", "default"), ("hier", "staged"), ("hier", "unfused"), ("topk", "default")])
def test_out_of_range_index_gradients(mode, path, dtype):
    """The gradients with out-of-range indices are those of the loss the forward returned: the
    offending pairs count as (latent 0, value 0) in dW, dvals and dbias of both losses, on every
    path (one of the pairs sits in a latent-0 group that also has regular pairs)."""
    B, K, F, D = 24, 16, 40, 256
    idx, W, v, b, t = make_inputs(B, K, F, D, dtype=dtype, seed=8)
    idx[3, 2] = F
    idx[5, 0] = -1
    idx[7, 9] = 1 << 40
    idx[2, 1] = 0           # a regular pair of latent 0
    idx2, v2 = idx.clone(), v.clone()
    for (r, c) in ((3, 2), (5, 0), (7, 9)):
        idx2[r, c] = 0
        v2[r, c] = 0
    flex.set_fused_training(path != "unfused")
    flex.set_hier_stage_bytes(STAGE_ALL if path == "staged" else None)
    try:
        got = _run_op(mode, (idx, W, v, b, t), 1.3)
    finally:
        flex.set_fused_training(True)
        flex.set_hier_stage_bytes(None)
    try:
        flex.check_index_flag()
    except IndexError:
        pass
    _check_against_oracle(mode, (idx2, W, v2, b, t), dtype, 1.3, got, ref_tols=False)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_fp16_weights_with_a_loss_scaling_upstream_gradient(mode):
    """fp16 leaves and grad_out = 2^16 (what a gradient scaler passes): the unit gradients, about
    2/(B*K*D), are far below fp16's range and must not be rounded to fp16 before the upstream
    gradient lifts them (the reference scales its fp32 gradients first, reference
    hierarchical_kernels.py:294-299)."""
    B, K, F, D = 64, 32, 224, 1024
    args = make_inputs(B, K, F, D, dtype=torch.float16, seed=21)
    grad_out = 65536.0
    got = _run_op(mode, args, grad_out)
    L, rW, rv, rb = oracle.loss_grads(MODES[mode], *args, grad_out=grad_out)
    # the scaled gradients are normal fp16 numbers: the plain fp16 bar applies, without any allowance
    assert float(np.abs(rW).max()) > 1e-4
    for name, g, r in (("dW", got[1], rW), ("dvals", got[2], rv), ("dbias", got[3], rb)):
        err = rel_err(g.float().cpu(), r)
        assert err <= 1e-3, f"{name}: {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_storage_offset_views(mode, dtype):
    """Contiguous tensors that start at an odd element of a larger buffer (a bias cut out of a flat
    parameter vector, a weight view): forward and backward work as in the reference, which
    addresses element-wise."""
    B, K, F, D = 16, 8, 40, 260
    args = make_inputs(B, K, F, D, dtype=dtype, seed=31)
    idx, W, v, b, t = _to_dev(args)

    def off_by_one(x):
        flat = torch.empty(x.numel() + 1, dtype=x.dtype, device=DEV)
        view = flat[1:].view(x.shape)
        view.copy_(x)
        assert view.is_contiguous() and view.data_ptr() % 16 != 0
        return view.requires_grad_()

    Wv, vv, bv = off_by_one(W), off_by_one(v), off_by_one(b)
    tv = off_by_one(t).detach()
    loss = FUSED[mode](idx, Wv, vv, bv, tv)
    loss.backward(torch.tensor(0.9, device=DEV))
    torch.cuda.synchronize()
    _check_against_oracle(mode, args, dtype, 0.9, (loss, Wv.grad, vv.grad, bv.grad), ref_tols=False)
    with torch.no_grad():
        loss2 = FUSED[mode](idx, Wv, vv, bv, tv)
    assert abs(loss2.item() - loss.item()) <= 1e-6 * abs(loss.item())


def test_topk_residual_precision_switch():
    """bf16 weights: the TopK backward gathers a bf16 copy of the residual by default (as the
    reference's backward receives it, reference topk_kernels.py:52); with the switch off it gathers
    the fp32 residual and dvals carry fp32 rounding only.  Both meet the bf16 bar."""
    B, K, F, D = 96, 32, 320, 1536
    args = make_inputs(B, K, F, D, dtype=torch.bfloat16, seed=23)
    L, rW, rv, rb = oracle.loss_grads(oracle.TOPK, *args, grad_out=0.7)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward("topk", idx, W, v, b, t)
    errs = {}
    for name, flags in (("bf16", 0), ("fp32", abi._lib.TOPK_BWD_FP32_RESIDUAL)):
        rc, dW, dv, db = abi.topk_backward(idx, W, v, resid, 0.7, dw_dtype=torch.float32, flags=flags)
        torch.cuda.synchronize()
        assert rc == 0
        errs[name] = (rel_err(dW.cpu(), rW), rel_err(dv.cpu(), rv), rel_err(db.cpu(), rb))
        print("[topk residual]", name, "dW %.2e dvals %.2e dbias %.2e" % errs[name], flush=True)
    assert errs["bf16"][0] < 1e-2 and errs["bf16"][1] < 1e-2
    assert errs["fp32"][0] < 1e-4 and errs["fp32"][1] < 1e-4 and errs["fp32"][2] < 1e-4
    # the python switch reaches the same two variants
    flex.set_topk_residual_bf16(False)
    try:
        got = _run_op("topk", args, 0.7)
    finally:
        flex.set_topk_residual_bf16(True)
    _check_against_oracle("topk", args, torch.bfloat16, 0.7, got, ref_tols=False)


@pytest.mark.parametrize("zipf,dtype", [(None, torch.bfloat16), (1.1, torch.bfloat16), (None, torch.float32)])
def test_dense_latents_hint_changes_no_bit(zipf, dtype):
    """Shapes with at most two pairs per latent reduce from a list of the latents ordered by pair
    count unless FLEXSAE_BWD_DENSE_LATENTS says most latents have pairs: the same results either way,
    bit for bit (training step and fused SGD update), and flexsae_hier_pair_stats counts the latents
    without pairs that the choice depends on."""
    import ctypes
    B, K, F, D = 256, 32, 5000, 384
    assert B * K <= 2 * F
    cpu_args = make_inputs(B, K, F, D, dtype=dtype, seed=37, zipf_s=zipf, unique=True)
    idx, W, v, b, t = _to_dev(cpu_args)
    DENSE = abi._lib.BWD_DENSE_LATENTS
    outs = {}
    for flags in (0, DENSE):
        rc, loss, dW, dv, db, ws = abi.hier_train(idx, W, v, b, t, dw_dtype=dtype, slice_cols=128, flags=flags,
                                                  keep_workspace=True)
        assert rc == 0, abi._lib.status_string(rc)
        outs[flags] = (loss, dW, dv, db)
        stats = torch.zeros(3, dtype=torch.int32, device=DEV)
        sh = abi.shape_of(idx, W, v, b.dtype, t.dtype)
        assert abi._lib.load().flexsae_hier_pair_stats(ctypes.byref(sh), abi.ptr(ws), abi.ptr(stats), abi.stream()) == 0
        counts = np.bincount(cpu_args[0].numpy().ravel(), minlength=F)
        assert [int(x) for x in stats.cpu()][::2] == [int((counts > 64).sum()), int((counts == 0).sum())]
    for a, c in zip(outs[0], outs[DENSE]):
        assert torch.equal(a, c)
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *cpu_args)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-4
    assert rel_err(outs[DENSE][1].double().cpu(), rW) <= tol and rel_err(outs[DENSE][2].cpu(), rv) <= tol
    # the in-place update
    upd = {}
    for flags in (0, DENSE):
        Wn = W.clone()
        rc, loss, dv, db = abi.hier_sgd_step(idx, Wn, v, b, t, 0.25, slice_cols=128, flags=flags)
        assert rc == 0, abi._lib.status_string(rc)
        upd[flags] = Wn
    assert torch.equal(upd[0], upd[DENSE])


def test_dense_latents_follow_the_previous_step():
    """Through the package: a shape with two pairs per latent starts with the row-count list; uniform
    indices (an eighth of the latents empty) drop it from the second step on, skewed ones keep it."""
    flex.set_dense_latents("auto")
    flex.set_hot_latents("off")  # (skewed indices would switch to the accumulators at the second step)
    B, K, F, D = 512, 16, 4096, 256
    try:
        for zipf, want_dense in ((None, True), (1.1, False)):
            cpu_args = make_inputs(B, K, F, D, dtype=torch.bfloat16, seed=38, zipf_s=zipf, unique=True)
            idx, W, v, b, t = _to_dev(cpu_args)
            flex.ops._hot_auto.clear()
            grads = []
            for step in range(3):
                assert flex.ops._use_dense_latents(B, K, F, D, torch.bfloat16, W.device) == (want_dense and step > 0)
                Wl = W.clone().requires_grad_()
                flex.triton_hierarchical_sae_loss(idx, Wl, v, b, t).backward()
                torch.cuda.synchronize()
                grads.append(Wl.grad)
            assert torch.equal(grads[0], grads[1]) and torch.equal(grads[1], grads[2])
            L, rW, _, _ = oracle.loss_grads(oracle.HIER, *cpu_args)
            assert rel_err(grads[2].double().cpu(), rW) <= 1e-2
    finally:
        flex.set_dense_latents(None)
        flex.set_hot_latents(None)


def test_topk_workspace_query_covers_both_residual_layouts():
    """bf16 weights, K = 512: the fp32-residual variant works on narrower tiles and needs more room
    for its per-tile shares of dvals than the bf16 one; the size query takes no flags and must
    cover both, so the same workspace serves either call."""
    B, K, F, D = 64, 512, 2048, 512
    args = make_inputs(B, K, F, D, dtype=torch.bfloat16, seed=29)
    L, rW, rv, rb = oracle.loss_grads(oracle.TOPK, *args, grad_out=1.0)
    idx, W, v, b, t = _to_dev(args)
    rc, loss, resid = abi.forward("topk", idx, W, v, b, t)
    assert rc == 0
    for flags, tol in ((0, 1e-2), (abi._lib.TOPK_BWD_FP32_RESIDUAL, 1e-4)):
        rc, dW, dv, db = abi.topk_backward(idx, W, v, resid, 1.0, dw_dtype=torch.float32, flags=flags)
        torch.cuda.synchronize()
        assert rc == 0, abi._lib.status_string(rc)
        assert rel_err(dW.cpu(), rW) < tol and rel_err(dv.cpu(), rv) < tol and rel_err(db.cpu(), rb) < 1e-4


def test_topk_target_gradient():
    args = make_inputs(16, 8, 40, 256, seed=2)
    idx, W, v, b, t = _to_dev(args)
    t.requires_grad_()
    W.requires_grad_()
    flex.triton_topk_sae_loss(idx, W, v, b, t).backward()
    tr = args[4].double().requires_grad_()
    oracle.torch_loss(oracle.TOPK, args[0], args[1].double(), args[2].double(), args[3].double(), tr,
                      compute_dtype=torch.float64).backward()
    assert rel_err(t.grad.cpu(), tr.grad) < 1e-4


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_non_contiguous_inputs(mode):
    idx, W, v, b, t = make_inputs(16, 8, 40, 256, seed=4)
    Wd = torch.empty(40, 512, device=DEV)[:, ::2]
    Wd.copy_(W)
    td = torch.empty(256, 16, device=DEV).t()
    td.copy_(t)
    assert not Wd.is_contiguous() and not td.is_contiguous()
    loss = FUSED[mode](idx.to(DEV), Wd, v.to(DEV), b.to(DEV), td)
    L, *_ = oracle.loss_grads(MODES[mode], idx, W, v, b, t, want_grads=False)
    assert abs(loss.item() - L) <= 1e-5 * abs(L)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_opcheck_and_compile(mode):
    args = _to_dev(make_inputs(16, 8, 40, 256, seed=6))
    idx, W, v, b, t = args
    W.requires_grad_()
    v.requires_grad_()
    b.requires_grad_()
    ops_ = ([torch.ops.flexsae_amd.hier_fwd, torch.ops.flexsae_amd.hier_train,
             torch.ops.flexsae_amd.hier_train_sliced] if mode == "hier" else [torch.ops.flexsae_amd.topk_fwd])
    for op in ops_:
        extra = (flex.ops.hier_train_stage(idx, W, v, b, t),) if op is torch.ops.flexsae_amd.hier_train else ()
        torch.library.opcheck(op, (idx, W, v, b, t, *extra),
                              test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    eager = FUSED[mode](idx, W, v, b, t)
    compiled = torch.compile(lambda *a: FUSED[mode](*a) * 2.0, fullgraph=True, backend="aot_eager")(idx, W, v, b, t)
    assert abs(compiled.item() - 2.0 * eager.item()) <= 1e-6 * abs(eager.item())
    compiled.backward()
    assert W.grad is not None and v.grad is not None and b.grad is not None
    if mode == "hier":  # the same with the contributions staged between forward and backward
        want = W.grad.clone()
        W.grad = None
        flex.set_hier_stage_bytes(STAGE_ALL)
        try:
            sliced = torch.compile(lambda *a: FUSED[mode](*a) * 2.0, fullgraph=True, backend="aot_eager")(idx, W, v, b, t)
            sliced.backward()
        finally:
            flex.set_hier_stage_bytes(None)
        assert abs(sliced.item() - compiled.item()) <= 1e-6 * abs(compiled.item())
        assert rel_err(W.grad.cpu(), want.cpu().numpy()) < 1e-5


def test_opcheck_of_every_op_with_all_checks():
    """torch.library.opcheck with its full default set of checks (schema, autograd registration,
    fake tensors, AOT dispatch with dynamic shapes) on every op of the package."""
    idx, W, v, b, t = _to_dev(make_inputs(16, 8, 40, 256, seed=6))
    ops = torch.ops.flexsae_amd
    g = torch.tensor(0.7, device=DEV)

    def leaves():
        return [x.clone().requires_grad_() for x in (W, v, b)]

    for op in (ops.hier_fwd, ops.topk_fwd, ops.hier_train_sliced):
        Wl, vl, bl = leaves()
        torch.library.opcheck(op, (idx, Wl, vl, bl, t))
    _, vl, bl = leaves()
    torch.library.opcheck(ops.hier_train_sliced, (idx, W, vl, bl, t, False))  # a frozen decoder
    # hier_train fills a scratch argument (the stage) next to its three outputs: the full default set
    # (like hier_sgd_step it mutates an argument, so it carries no autograd formula of its own: the
    # staged step's autograd glue sits above it and is covered by the parity tests)
    torch.library.opcheck(ops.hier_train, (idx, W, v, b, t, flex.ops.hier_train_stage(idx, W, v, b, t)))
    _, resid_h = ops.hier_fwd(idx, W, v, b, t)
    _, resid_t = ops.topk_fwd(idx, W, v, b, t)
    torch.library.opcheck(ops.hier_bwd, (g, idx, W, v, resid_h))
    torch.library.opcheck(ops.topk_bwd, (g, idx, W, v, resid_t))
    stage = flex.ops.hier_train_stage(idx, W, v, b, t)
    ops.hier_train(idx, W, v, b, t, stage)
    torch.library.opcheck(ops.hier_finish, (g, idx, W, v, stage))
    torch.library.opcheck(ops.scale_by, (W, g))
    torch.library.opcheck(ops.scale_, (W.clone(), g))
    torch.library.opcheck(ops.hier_sgd_step, (idx, W.clone(), v, b, t, g))  # mutates its weight argument


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_compile_with_the_default_backend(mode):
    """torch.compile(fullgraph=True) with the default backend (inductor) around the fused loss, as
    a caller compiling the training step would (reference example.py:15 compiles its competitor):
    same loss and gradients as eager."""
    args = make_inputs(32, 16, 96, 512, seed=9)
    idx, W, v, b, t = _to_dev(args)
    leaves_e = [x.clone().requires_grad_() for x in (W, v, b)]
    leaves_c = [x.clone().requires_grad_() for x in (W, v, b)]

    def fn(i, w, vv, bb, tt):
        return FUSED[mode](i, w, vv * 1.5, bb, tt) * 2.0 + 1.0

    eager = fn(idx, *leaves_e, t)
    eager.backward()
    torch._dynamo.reset()
    compiled = torch.compile(fn, fullgraph=True)(idx, *leaves_c, t)
    compiled.backward()
    torch.cuda.synchronize()
    assert abs(compiled.item() - eager.item()) <= 1e-6 * abs(eager.item())
    for ge, gc in zip(leaves_e, leaves_c):
        assert gc.grad is not None and rel_err(gc.grad.cpu(), ge.grad.cpu().numpy()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("order", ["topk_first", "hier_first"])
@pytest.mark.parametrize("fused", ["sliced", "staged", "unfused"])
def test_shared_pair_list_changes_nothing(order, fused, dtype):
    """Inside shared_pair_list() the second loss on the same indices reuses the first one's pair
    list; loss and gradients stay bit-identical to the unshared calls."""
    args = make_inputs(64, 16, 300, 512, dtype=dtype, seed=77)
    modes = ["topk", "hier"] if order == "topk_first" else ["hier", "topk"]
    flex.set_fused_training(fused != "unfused")
    flex.set_hier_stage_bytes(STAGE_ALL if fused == "staged" else None)
    try:
        plain = {m: _run_op(m, args, 0.8) for m in modes}
        shared = {}
        idx, W, v, b, t = _to_dev(args)
        with flex.shared_pair_list():
            for m in modes:
                Wm, vm, bm = (x.clone().requires_grad_() for x in (W, v, b))
                loss = FUSED[m](idx, Wm, vm, bm, t)  # the same indices tensor for both losses
                loss.backward(torch.tensor(0.8, device=DEV))
                shared[m] = (loss, Wm.grad, vm.grad, bm.grad)
            assert len(flex.ops._pair_cache) == 1
        assert flex.ops._pair_cache is None
    finally:
        flex.set_fused_training(True)
        flex.set_hier_stage_bytes(None)
    torch.cuda.synchronize()
    for m in modes:
        for a, c in zip(plain[m], shared[m]):
            assert torch.equal(a, c), m


def test_pair_list_import_through_the_c_abi():
    """flexsae_csr_build -> flexsae_hier_import_pair_list -> flexsae_hier_bwd(REUSE_PAIR_LIST) equals the
    plain call, and the layout query points at the list a plain call leaves in its workspace."""
    import ctypes
    from flexsae_amd import _lib
    lib = _lib.load()
    args = _to_dev(make_inputs(40, 24, 90, 640, seed=5))
    idx, W, v, b, t = args
    _, _, resid = abi.forward("hier", *args)
    rc, dW0, dv0, db0 = abi.hier_backward(idx, W, v, resid, 1.25)
    assert rc == 0
    sh = abi.shape_of(idx, W, v)
    rc, begin, mp = abi.csr_build(idx, sh.F)
    assert rc == 0
    nbytes = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), 0)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    assert lib.flexsae_hier_import_pair_list(ctypes.byref(sh), abi.ptr(begin), abi.ptr(mp), abi.ptr(ws), nbytes,
                                             abi.stream()) == 0
    dW = torch.full_like(dW0, float("nan"))
    dv = torch.full_like(dv0, float("nan"))
    db = torch.full_like(db0, float("nan"))
    g = torch.tensor([1.25], dtype=torch.float32, device=DEV)
    rc = lib.flexsae_hier_bwd(ctypes.byref(sh), abi.ptr(idx), abi.ptr(W), abi.ptr(v), abi.ptr(resid), abi.ptr(g),
                              abi.ptr(dW), abi.DT[torch.float32], abi.ptr(dv), abi.ptr(db), abi.ptr(ws), nbytes,
                              _lib.BWD_REUSE_PAIR_LIST, None, abi.stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(dW, dW0) and torch.equal(dv, dv0) and torch.equal(db, db0)
    ob, om = ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.flexsae_hier_pair_list_layout(ctypes.byref(sh), ctypes.byref(ob), ctypes.byref(om)) == 0
    n_pairs = idx.numel()
    assert torch.equal(ws[ob.value: ob.value + (sh.F + 1) * 4].view(torch.int32), begin)
    assert torch.equal(ws[om.value: om.value + n_pairs * 4].view(torch.int32), mp)


@pytest.mark.parametrize("mode", ["hier", "topk"])
def test_int32_indices_are_accepted(mode):
    args = make_inputs(32, 8, 120, 256, seed=12)
    ref = _run_op(mode, args, 1.0)
    idx, W, v, b, t = _to_dev(args)
    W.requires_grad_()
    loss = FUSED[mode](idx.to(torch.int32), W, v, b, t)
    loss.backward()
    assert torch.equal(loss, ref[0]) and torch.equal(W.grad, ref[1])


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes(seed):
    """Seeded random shapes and dtypes, both losses, against the oracle: K below/above the 64-step
    and 128-step limits of the register-resident paths, D with every vector width, F from a
    handful of hot latents to mostly unused ones."""
    rng = np.random.default_rng(1000 + seed)
    B = int(rng.integers(1, 70))
    K = int(rng.choice([1, 2, 3, 7, 8, 16, 31, 33, 64, 65, 100, 128, 129, 140]))
    F = int(rng.choice([1, 2, 5, 40, 300, 2000]))
    D = int(rng.choice([1, 2, 4, 6, 8, 62, 64, 100, 128, 130, 256, 260, 520, 700]))
    dtype = [torch.float32, torch.bfloat16, torch.float16][seed % 3]
    grad_out = float(rng.normal())
    _announce("random", seed, (B, K, F, D), dtype, grad_out)
    args = make_inputs(B, K, F, D, dtype=dtype, seed=seed)
    flex.set_hier_stage_bytes(STAGE_ALL if seed % 2 else None)  # odd seeds: contributions staged
    try:
        for mode in ("hier", "topk"):
            got = _run_op(mode, args, grad_out)
            _check_against_oracle(mode, args, dtype, grad_out, got, ref_tols=False)
    finally:
        flex.set_hier_stage_bytes(None)


@pytest.mark.parametrize("mode", ["hier", "hier_staged", "topk"])
def test_step_can_be_captured_in_a_graph(mode):
    """Forward + backward recorded into a HIP graph (no memset nodes, no synchronisation, no
    allocation outside torch's graph pool) and replayed with new input values, with eager work
    between the replays; every replay must equal the eager result on the same values."""
    args = make_inputs(48, 16, 200, 512, dtype=torch.bfloat16, seed=3)
    idx, W, v, b, t = _to_dev(args)
    W.requires_grad_()
    v.requires_grad_()
    b.requires_grad_()
    loss_name = mode.split("_")[0]
    fn = FUSED[loss_name]
    flex.set_hier_stage_bytes(STAGE_ALL if mode == "hier_staged" else None)
    try:
        _graph_capture_body(loss_name, fn, idx, W, v, b, t)
    finally:
        flex.set_hier_stage_bytes(None)


def _graph_capture_body(mode, fn, idx, W, v, b, t):
    def step():
        W.grad = v.grad = b.grad = None
        loss = fn(idx, W, v, b, t)
        loss.backward()
        return loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    W.grad = v.grad = b.grad = None
    with torch.cuda.graph(graph):
        static_loss = fn(idx, W, v, b, t)
        static_loss.backward()
    for trial in range(3):
        new = make_inputs(48, 16, 200, 512, dtype=torch.bfloat16, seed=100 + trial)
        with torch.no_grad():
            for dst, src in zip((idx, W, v, b, t), new):
                dst.copy_(src.to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = (static_loss.clone(), W.grad.clone(), v.grad.clone(), b.grad.clone())
        ref = _run_op(mode, new, 1.0)  # eager work between the replays
        for a, c in zip(got, ref):
            assert torch.equal(a, c), (mode, trial)
