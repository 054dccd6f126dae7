"""Hot-latent accumulators of the training step (FLEXSAE_BWD_HOT_LATENTS), through the C ABI.

The most frequent latents of a batch are summed in LDS accumulators (32-bit fixed point, one
exponent per block of 128 rows) instead of being staged pair by pair.  Checked here: parity with the
oracle on skewed indices (every K variant of the kernel, bf16 and fp16 weights, a ragged last row
block, more long latents than accumulator rows), that loss / dvals / dbias are the bits of the plain
step, that latents with a repeated row stay cold (duplicates: dW bit-identical to the plain step),
the deferred second pass (forced by FLEXSAE_BWD_HOT_NO_HEADROOM), bit-identical dW for every slice
width and from run to run, and the fused SGD update.
"""
import ctypes

import numpy as np
import pytest
import torch

import abi
from flexsae_amd import _lib
import oracle
from helpers import make_inputs, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
HOT = _lib.BWD_HOT_LATENTS


def _dev(args):
    return tuple(x.to(DEV) for x in args)


def _supported(idx, W, v, b, t):
    sh = abi.shape_of(idx, W, v, b.dtype, t.dtype)
    return bool(_lib.load().flexsae_hier_hot_latents_supported(ctypes.byref(sh)))


def _check_vs_oracle(cpu_args, dW, dv, db, loss, tol):
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *cpu_args)
    assert abs(loss.item() - L) <= max(tol * 1e-1, 1e-5) * abs(L)
    assert rel_err(dv.cpu(), rv) <= tol
    assert rel_err(db.cpu(), rb) <= tol
    got, ref = dW.double().cpu(), torch.from_numpy(rW)
    assert rel_err(got, ref) <= tol
    # element by element too: |got - ref| <= tol |ref| + tol max|ref|
    assert float(((got - ref).abs() - tol * ref.abs()).max()) <= tol * float(ref.abs().max())
    return ref


@pytest.mark.parametrize("shape,dtype,zipf", [
    ((300, 64, 2000, 512), torch.bfloat16, 1.1),     # ragged last row block, full 64-step kernel
    ((256, 32, 1500, 264), torch.bfloat16, 1.2),     # 32 steps, D not a whole tile
    ((200, 16, 900, 128), torch.bfloat16, 1.3),      # 16 steps
    ((260, 40, 1200, 384), torch.bfloat16, 1.1),     # K below the kernel's bound (per-step tests)
    ((384, 64, 1800, 256), torch.float16, 1.1),      # fp16 weights: fp32 contributions, fp32 dW
    ((2048, 64, 1000, 128), torch.bfloat16, 0.3),    # more long latents than accumulator rows
    ((300, 64, 40000, 1536), torch.bfloat16, 1.1),   # most latents without a pair (the sparse reduction and its zero pass)
    ((256, 32, 30000, 264), torch.bfloat16, 1.2),    # the same with a ragged last tile
    ((384, 64, 50000, 256), torch.float16, 1.1),     # ... and an fp32 gradient of fp16 weights
])
def test_hot_latents_match_the_oracle(shape, dtype, zipf):
    print("[case] hot", shape, dtype, zipf, flush=True)
    cpu_args = make_inputs(*shape, dtype, seed=31, zipf_s=zipf, sort_vals=True, w_std=0.3)
    args = _dev(cpu_args)
    assert _supported(*args)
    dw_dtype = torch.float32 if dtype == torch.float16 else dtype
    rc0, loss0, dW0, dv0, db0 = abi.hier_train(*args, dw_dtype=dw_dtype, slice_cols=256)
    rc, loss, dW, dv, db, ws = abi.hier_train(*args, dw_dtype=dw_dtype, slice_cols=256, flags=HOT, keep_workspace=True)
    assert rc0 == 0 and rc == 0, (_lib.status_string(rc0), _lib.status_string(rc))
    n_hot, n_cand, n_cold_long, threshold, deferred = abi.hot_stats(*args, ws)
    counts = np.bincount(cpu_args[0].numpy().ravel(), minlength=shape[2])
    n_long = int((counts > 64).sum())
    assert n_hot == n_cand == min(n_long, int((counts > threshold).sum())) and 0 < n_hot <= 288  # per-row unique indices
    assert n_cold_long == n_long - n_hot and deferred == 0
    if n_long > 288:  # the threshold is the 289th largest pair count
        assert threshold == int(np.sort(counts)[-289])
    # the hot latents change nothing but dW (and the summation order of dbias)
    assert torch.equal(loss, loss0) and torch.equal(dv, dv0)
    # dbias: the same values summed in another fixed order (per block of 128 rows on chip)
    assert rel_err(db.cpu(), db0.cpu()) <= 2e-6
    assert n_long > 0, "the case has no frequent latent"
    assert not torch.equal(dW, dW0), "the hot path was not taken"
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-4
    ref = _check_vs_oracle(cpu_args, dW, dv, db, loss, tol)
    # rows of the frequent latents: fixed point with 23 bits below the block's bound is far more
    # exact than one bf16 rounding per contribution
    hot_rows = torch.from_numpy(np.argsort(-counts)[:16].copy())
    e_hot = rel_err(dW[hot_rows.to(DEV)].double().cpu(), ref[hot_rows])
    e_plain = rel_err(dW0[hot_rows.to(DEV)].double().cpu(), ref[hot_rows])
    assert e_hot <= (4e-3 if dtype == torch.bfloat16 else 2e-5), (e_hot, e_plain)


def test_repeated_rows_keep_a_latent_cold():
    """randint indices on few latents: every latent is frequent and nearly every one is repeated
    inside some row, so none may be summed in the accumulators: dW is the plain step's, bit for bit."""
    print("[case] hot duplicates", flush=True)
    args = _dev(make_inputs(192, 64, 96, 256, torch.bfloat16, seed=5))
    rc0, _, dW0, _, _ = abi.hier_train(*args, dw_dtype=torch.bfloat16)
    rc, _, dW, _, _ = abi.hier_train(*args, dw_dtype=torch.bfloat16, flags=HOT)
    assert rc0 == 0 and rc == 0
    assert torch.equal(dW, dW0)


def test_deferred_rows_and_reproducibility():
    """With the block exponent set 8 bits low most rows exceed it, are left out of the first pass
    and walked again after the exponent has been raised: still the oracle's dW, the same bits on
    every run and for every slice width; and so for the normal headroom."""
    print("[case] hot deferred", flush=True)
    cpu_args = make_inputs(300, 64, 2000, 512, torch.bfloat16, seed=32, zipf_s=1.1, sort_vals=True, w_std=0.3)
    # rows of very different magnitude: the later rows of every block dwarf its first ones
    scale = torch.ones(300)
    scale[40::3] = 64.0
    cpu_args = (cpu_args[0], cpu_args[1], cpu_args[2], cpu_args[3], (cpu_args[4].float() * scale[:, None]).to(torch.bfloat16))
    args = _dev(cpu_args)
    for extra in (0, _lib.BWD_HOT_NO_HEADROOM):
        outs, dbs = [], []
        for cols in (128, 256, 512, 128):
            rc, loss, dW, dv, db, ws = abi.hier_train(*args, dw_dtype=torch.bfloat16, slice_cols=cols, flags=HOT | extra,
                                                      keep_workspace=True)
            assert rc == 0
            deferred = abi.hot_stats(*args, ws)[4]
            print("deferred walks", deferred, "of", 300 * 4, flush=True)
            assert deferred > (300 if extra else 0)
            outs.append(dW)
            dbs.append(db)
        for o in outs[1:]:
            assert torch.equal(o, outs[0])
        for o in dbs[1:]:  # dbias too is the same bits for every slice width
            assert torch.equal(o, dbs[0])
        _check_vs_oracle(cpu_args, outs[0], dv, db, loss, 1e-2)


def test_pair_list_and_hot_tables_reused():
    """A second call on the same workspace may keep the pair list (FLEXSAE_BWD_REUSE_PAIR_LIST: the hot
    tables are rebuilt from it) and the hot tables too (FLEXSAE_BWD_REUSE_HOT_TABLES): the same bits
    either way, also for other values and targets on the same indices."""
    print("[case] hot reuse", flush=True)
    cpu_args = make_inputs(300, 64, 2000, 512, torch.bfloat16, seed=34, zipf_s=1.1, sort_vals=True, w_std=0.3)
    idx, W, v, b, t = _dev(cpu_args)
    rc, loss0, dW0, dv0, db0, ws = abi.hier_train(idx, W, v, b, t, dw_dtype=torch.bfloat16, slice_cols=256, flags=HOT,
                                                   keep_workspace=True)
    assert rc == 0 and abi.hot_stats(idx, W, v, b, t, ws)[0] > 0
    v2, t2 = (v.float() * 0.5 + 0.1).to(v.dtype), (t.float() * 1.5).to(t.dtype)
    rc, loss1, dW1, dv1, db1 = abi.hier_train(idx, W, v2, b, t2, dw_dtype=torch.bfloat16, slice_cols=256, flags=HOT)
    assert rc == 0
    for reuse in (_lib.BWD_REUSE_PAIR_LIST, _lib.BWD_REUSE_PAIR_LIST | _lib.BWD_REUSE_HOT_TABLES):
        for (vv, tt), want in (((v, t), (loss0, dW0, dv0, db0)), ((v2, t2), (loss1, dW1, dv1, db1))):
            rc, loss, dW, dv, db = abi.hier_train(idx, W, vv, b, tt, dw_dtype=torch.bfloat16, slice_cols=256,
                                                  flags=HOT | reuse, workspace=ws)
            assert rc == 0, _lib.status_string(rc)
            assert torch.equal(loss, want[0]) and torch.equal(dW, want[1])
            assert torch.equal(dv, want[2]) and torch.equal(db, want[3])


def test_hot_latents_under_a_shared_pair_list():
    """Through the package: both losses inside shared_pair_list() with the hot path forced on give
    the gradients of separate calls, bit for bit."""
    import flexsae_amd as flex
    print("[case] hot shared pair list", flush=True)
    cpu_args = make_inputs(512, 64, 3000, 512, torch.bfloat16, seed=35, zipf_s=1.1, sort_vals=True, w_std=0.3)

    def grads(shared):
        idx, W, v, b, t = _dev(cpu_args)
        W.requires_grad_(); v.requires_grad_(); b.requires_grad_()
        import contextlib
        with (flex.shared_pair_list() if shared else contextlib.nullcontext()):
            (flex.triton_hierarchical_sae_loss(idx, W, v, b, t) + flex.triton_topk_sae_loss(idx, W, v, b, t)).backward()
        return W.grad, v.grad, b.grad

    flex.set_hot_latents("on")
    try:
        a, b_ = grads(False), grads(True)
    finally:
        flex.set_hot_latents("auto")
    for x, y in zip(a, b_):
        assert torch.equal(x, y)
    # and the hot path was what ran: differs from the plain step in dW only by rounding
    flex.set_hot_latents("off")
    try:
        c = grads(False)
    finally:
        flex.set_hot_latents("auto")
    assert not torch.equal(a[0], c[0]) and rel_err(a[0].float().cpu(), c[0].float().cpu()) < 1e-2
    assert torch.equal(a[1], c[1])


def test_hot_step_in_a_graph():
    """The step with the hot path forced on, recorded into a HIP graph and replayed with other
    indices (another set of frequent latents) and values, eager work between the replays: every
    replay equals the eager step on the same inputs, bit for bit.  Selection, marking and the
    accumulators' exponents all live on the device, so nothing of them is frozen into the graph."""
    import flexsae_amd as flex
    print("[case] hot graph", flush=True)
    shape = (300, 64, 2000, 512)
    mk = lambda seed: make_inputs(*shape, torch.bfloat16, seed=seed, zipf_s=1.1, sort_vals=True, w_std=0.3)
    idx, W, v, b, t = _dev(mk(40))
    W.requires_grad_(); v.requires_grad_(); b.requires_grad_()

    def step():
        W.grad = v.grad = b.grad = None
        loss = flex.triton_hierarchical_sae_loss(idx, W, v, b, t)
        loss.backward()
        return loss

    flex.set_hot_latents("on")
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        W.grad = v.grad = b.grad = None
        with torch.cuda.graph(graph):
            static_loss = flex.triton_hierarchical_sae_loss(idx, W, v, b, t)
            static_loss.backward()
        for trial in range(3):
            new = mk(41 + trial)
            with torch.no_grad():
                for dst, src in zip((idx, W, v, b, t), new):
                    dst.copy_(src.to(DEV))
            graph.replay()
            torch.cuda.synchronize()
            got = (static_loss.clone(), W.grad.clone(), v.grad.clone(), b.grad.clone())
            i2, W2, v2, b2, t2 = _dev(new)  # eager work between the replays
            W2.requires_grad_(); v2.requires_grad_(); b2.requires_grad_()
            loss2 = flex.triton_hierarchical_sae_loss(i2, W2, v2, b2, t2)
            loss2.backward()
            for a, c in zip(got, (loss2.detach(), W2.grad, v2.grad, b2.grad)):
                assert torch.equal(a, c), trial
            L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *new)
            assert rel_err(got[1].double().cpu(), torch.from_numpy(rW)) <= 1e-2
    finally:
        flex.set_hot_latents("auto")


def test_sgd_update_with_hot_latents():
    print("[case] hot sgd", flush=True)
    cpu_args = make_inputs(300, 64, 2000, 512, torch.bfloat16, seed=33, zipf_s=1.1, sort_vals=True, w_std=0.3)
    idx, W, v, b, t = _dev(cpu_args)
    step = 0.37
    Wn = W.clone()
    rc, loss, dv, db = abi.hier_sgd_step(idx, Wn, v, b, t, step, slice_cols=256, flags=HOT)
    assert rc == 0, _lib.status_string(rc)
    L, rW, rv, rb = oracle.loss_grads(oracle.HIER, *cpu_args)
    want = cpu_args[1].double() - step * torch.from_numpy(rW)
    touched = torch.from_numpy(np.bincount(cpu_args[0].numpy().ravel(), minlength=2000) > 0)
    # update = step * dW: compare the change, within bf16's rounding of the new weights
    assert rel_err(Wn.double().cpu()[touched], want[touched]) <= 4e-3
    assert torch.equal(Wn.cpu()[~touched], cpu_args[1][~touched])
    assert abs(loss.item() - L) <= 1e-3 * abs(L) and rel_err(dv.cpu(), rv) <= 1e-2


def test_auto_mode_follows_the_previous_step():
    """"auto": the first step of a shape runs the plain kernel and leaves the skew of its indices in
    pinned memory; the next step takes the accumulators for skewed indices and stays plain for
    uniform ones.  Gradients match the oracle either way."""
    import flexsae_amd as flex

    print("[case] hot auto", flush=True)
    flex.set_hot_latents("auto")
    try:
        for zipf, want_hot in ((1.1, True), (None, False)):
            shape = (300, 64, 2000, 512) if zipf else (300, 64, 60000, 512)
            cpu_args = make_inputs(*shape, torch.bfloat16, seed=34, zipf_s=zipf, unique=zipf is None, sort_vals=True,
                                   w_std=0.3)
            idx, W, v, b, t = _dev(cpu_args)
            key = flex.ops._hot_key(W.device, *shape, torch.bfloat16)
            grads = []
            for step in range(3):
                Wl = W.clone().requires_grad_()
                loss = flex.triton_hierarchical_sae_loss(idx, Wl, v, b, t)
                loss.backward()
                torch.cuda.synchronize()
                grads.append(Wl.grad)
                # after a synchronisation the measurement is there for the next call to pick up
                assert flex.ops._use_hot_latents(*shape, torch.bfloat16, W.device) == want_hot, (zipf, step)
            assert flex.ops._hot_auto[key]["hot"] == want_hot
            L, rW, _, _ = oracle.loss_grads(oracle.HIER, *cpu_args)
            assert abs(loss.item() - L) <= 1e-3 * abs(L)
            for g in grads:
                assert rel_err(g.double().cpu(), rW) <= 1e-2
            if want_hot:  # the first step ran the plain kernel, the later ones the accumulators
                assert not torch.equal(grads[0], grads[1]) and torch.equal(grads[1], grads[2])
            else:
                assert torch.equal(grads[0], grads[1]) and torch.equal(grads[1], grads[2])
    finally:
        flex.set_hot_latents(None)
