"""flexsae_hier_fwd_static, the entry point that allocates nothing (its loss partials live in a
static device array): bit-identical to flexsae_hier_fwd on two calls in a row, the second one on
a smaller input, so that whatever the first call left in the shared array cannot leak into the
second result."""
import ctypes

import pytest
import torch

from flexsae_amd import _lib
from tests import abi
from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu


def _outputs(B, D, dev):
    """Caller-owned outputs, filled with NaN so that an element the call does not write shows."""
    return (torch.full((1,), float("nan"), dtype=torch.float32, device=dev),
            torch.full((B, D), float("nan"), dtype=torch.float32, device=dev))


def _static_forward(sh, indices, weight, vals, bias, target, loss, resid, stream, flag=None):
    """The entry point through ctypes alone: no torch call between the arguments and the launch."""
    return _lib.load().flexsae_hier_fwd_static(ctypes.byref(sh), abi.ptr(indices), abi.ptr(weight), abi.ptr(vals),
                                               abi.ptr(bias), abi.ptr(target), abi.ptr(loss), abi.ptr(resid),
                                               abi.ptr(flag), stream)


def test_static_forward_matches_workspace_forward_twice():
    dev = torch.device("cuda", 0)
    cases = [((96, 64, 288, 2048), torch.bfloat16, 11), ((16, 16, 64, 512), torch.float32, 12),
             ((7, 5, 300, 260), torch.float16, 13)]
    for (B, K, F, D), dtype, seed in cases:  # later cases are smaller than the first
        idx, W, v, b, t = (x.to(dev) for x in make_inputs(B, K, F, D, dtype, seed=seed))
        rc_ref, loss_ref, resid_ref = abi.forward("hier", idx, W, v, b, t)
        assert rc_ref == 0
        sh = abi.shape_of(idx, W, v, b.dtype, t.dtype)
        stream = abi.stream()
        # every output is allocated before the measured window; the first call also resolves the
        # per-device address of the static array
        loss, resid = _outputs(B, D, dev)
        loss2, resid2 = _outputs(B, D, dev)
        rc = _static_forward(sh, idx, W, v, b, t, loss, resid, stream)
        assert rc == 0, _lib.status_string(rc)
        torch.cuda.synchronize()
        assert torch.equal(loss, loss_ref), (B, K, F, D, loss.item(), loss_ref.item())
        assert torch.equal(resid, resid_ref)
        assert torch.isfinite(loss).all()
        # a second call on the same input, bracketed: the device's free memory and torch's own
        # allocation counters are exactly what they were (the call reaches the device through
        # ctypes only), and the bits are the same again
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        allocated_before, reserved_before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        rc2 = _static_forward(sh, idx, W, v, b, t, loss2, resid2, stream)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_allocated() == allocated_before and torch.cuda.memory_reserved() == reserved_before
        assert rc2 == 0 and torch.equal(loss2, loss_ref) and torch.equal(resid2, resid_ref)


def test_static_forward_rejects_what_does_not_fit():
    dev = torch.device("cuda", 0)
    lib = _lib.load()
    # B * ceil(D/64) * 4 bytes beyond the 16 MiB array: rejected before anything is launched
    B, K, F, D = 70000, 1, 8, 64 * 64
    sh = _lib.Shape(B, K, F, D, _lib.F32, _lib.F32, _lib.F32, _lib.F32)
    assert lib.flexsae_fwd_workspace_bytes(ctypes.byref(sh)) > (16 << 20)
    x = torch.zeros(8, device=dev)
    rc = lib.flexsae_hier_fwd_static(ctypes.byref(sh), abi.ptr(x), abi.ptr(x), abi.ptr(x), abi.ptr(x), abi.ptr(x),
                                     abi.ptr(x), abi.ptr(x), None, abi.stream())
    assert rc == _lib.ERR_SCRATCH_LIMIT
    assert "static scratch" in _lib.status_string(rc)
