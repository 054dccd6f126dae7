"""Host-side logic of the python layer (no GPU): validation, public names, fake kernels, the
eager torch definitions, and that nothing in the package touches the oracle."""
import os
import re

import pytest
import torch

import flexsae_amd as flex
import oracle
from flexsae_amd import ops
from helpers import make_inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_public_names_match_the_reference_package():
    # reference torch-ext/flex_sae/__init__.py:12-18
    for name in ("__kernel_metadata__", "topk_sae_loss", "triton_topk_sae_loss", "hierarchical_sae_loss",
                 "triton_hierarchical_sae_loss"):
        assert name in flex.__all__ and hasattr(flex, name)


@pytest.mark.parametrize("fn", [flex.triton_topk_sae_loss, flex.triton_hierarchical_sae_loss])
def test_fused_ops_fail_loudly_without_a_gpu_tensor(fn):
    args = make_inputs(4, 8, 16, 64)
    with pytest.raises(RuntimeError, match="AMD GPU only"):
        fn(*args)


def test_validation_errors():
    idx, W, v, b, t = make_inputs(4, 8, 16, 64)
    with pytest.raises(TypeError):
        ops._validate(idx.int(), W, v, b, t)
    with pytest.raises(TypeError):
        ops._validate(idx, W.double(), v, b, t)
    with pytest.raises(ValueError):
        ops._validate(idx, W, v[:, :4], b, t)
    with pytest.raises(ValueError):
        ops._validate(idx, W, v, b[:32], t)
    with pytest.raises(ValueError):
        ops._validate(idx[:0], W, v[:0], b, t[:0])
    with pytest.raises(ValueError):
        ops._validate(idx.flatten(), W, v, b, t)


@pytest.mark.parametrize("mode,fn", [(oracle.TOPK, flex.topk_sae_loss), (oracle.HIER, flex.hierarchical_sae_loss)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_eager_definitions_agree_with_oracle(mode, fn, dtype):
    args = make_inputs(16, 16, 64, 128, dtype=dtype)
    L, *_ = oracle.loss_grads(mode, *args, want_grads=False)
    got = fn(*args)
    assert got.dtype == torch.float32 and got.dim() == 0
    assert abs(got.item() - L) <= 2e-6 * abs(L)


@pytest.mark.parametrize("name", ["hier_fwd", "topk_fwd"])
def test_fake_kernels_give_shapes_and_dtypes(name):
    op = getattr(torch.ops.flexsae_amd, name)
    meta = lambda *s, dt=torch.bfloat16: torch.empty(*s, dtype=dt, device="meta")
    loss, resid = op(meta(32, 8, dt=torch.int64), meta(100, 256), meta(32, 8), meta(256), meta(32, 256))
    assert loss.shape == () and loss.dtype == torch.float32
    assert resid.shape == (32, 256) and resid.dtype == torch.float32
    bop = getattr(torch.ops.flexsae_amd, name.replace("fwd", "bwd"))
    dW, dv, db = bop(torch.empty((), dtype=torch.float32, device="meta"), meta(32, 8, dt=torch.int64),
                     meta(100, 256), meta(32, 8), resid)
    assert dW.shape == (100, 256) and dW.dtype == torch.bfloat16
    assert dv.shape == (32, 8) and dv.dtype == torch.float32
    assert db.shape == (256,) and db.dtype == torch.float32


def test_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flexsae_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
                assert "sae_oracle" not in text, f
