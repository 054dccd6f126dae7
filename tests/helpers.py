"""Seeded input builders shared by the CPU and GPU test modules."""
import torch

SEED = 1234  # the reference's test seed (reference tests/test_setup.py:3)

# The reference's shape matrix (B, K, F, D) -- reference tests/test_setup.py:5-32.
PARAMS = [
    (16, 16, 64, 512), (16, 32, 96, 768), (16, 64, 128, 1024), (32, 16, 128, 512),
    (32, 32, 160, 768), (32, 64, 192, 1024), (48, 32, 176, 1024), (48, 64, 224, 1280),
    (64, 16, 192, 768), (64, 32, 224, 1024), (64, 128, 256, 2048), (80, 32, 240, 1280),
    (80, 64, 256, 1536), (96, 32, 256, 1536), (96, 64, 288, 2048), (96, 128, 320, 3072),
    (112, 64, 320, 2048), (112, 128, 352, 2560), (128, 32, 256, 1024), (128, 64, 320, 1536),
    (128, 128, 384, 3072), (160, 64, 320, 1536), (160, 128, 384, 2560), (192, 64, 384, 2048),
    (192, 128, 448, 3072), (192, 256, 512, 4096),
]

# assert_close tolerances per dtype -- reference tests/test_setup.py:35-39.
DTYPE_TO_TOLS = {
    torch.float32: {"atol": 1e-4, "rtol": 1e-3},
    torch.bfloat16: {"atol": 1e-2, "rtol": 1e-2},
    torch.float16: {"atol": 1e-3, "rtol": 1e-3},
}

# Parity bar of this build: normwise relative error per dtype (loss, gradients).
REL_TOL = {
    torch.float32: (1e-5, 1e-4),
    torch.bfloat16: (1e-2, 1e-2),
    torch.float16: (1e-3, 1e-3),
}


def make_inputs(B, K, F, D, dtype=torch.float32, seed=SEED, unique=False, w_std=1.0,
                sort_vals=False, zipf_s=None):
    """CPU-generated inputs in the order indices, vals, weight, bias, target.

    ``unique``: per-row indices without replacement; ``zipf_s``: per-row unique
    indices with rank probabilities ~ r^-s mapped through a random permutation of F.
    """
    g = torch.Generator().manual_seed(seed)
    if zipf_s is not None:
        logp = -zipf_s * torch.log(torch.arange(1, F + 1, dtype=torch.float64))
        perm = torch.randperm(F, generator=g)
        idx = torch.empty(B, K, dtype=torch.long)
        step = max(1, (1 << 24) // F)
        for b0 in range(0, B, step):
            n = min(step, B - b0)
            u = torch.rand(n, F, generator=g, dtype=torch.float64).clamp_min_(1e-300)
            gumbel = -torch.log(-torch.log(u))
            idx[b0:b0 + n] = perm[(logp + gumbel).topk(K, dim=1).indices]
    elif unique:
        idx = torch.empty(B, K, dtype=torch.long)
        step = max(1, (1 << 24) // F)
        for b0 in range(0, B, step):
            n = min(step, B - b0)
            idx[b0:b0 + n] = torch.rand(n, F, generator=g).topk(K, dim=1).indices
    else:
        idx = torch.randint(0, F, (B, K), generator=g, dtype=torch.long)
    vals = torch.randn(B, K, generator=g).abs()
    if sort_vals:
        vals = vals.sort(dim=1, descending=True).values
    weight = torch.randn(F, D, generator=g) * w_std
    bias = torch.randn(D, generator=g)
    target = torch.randn(B, D, generator=g)
    return idx, weight.to(dtype), vals.to(dtype), bias.to(dtype), target.to(dtype)


def rel_err(a, b):
    """Normwise relative error ||a-b|| / ||b|| in float64 (0 when both are zero)."""
    a = torch.as_tensor(a, dtype=torch.float64).flatten()
    b = torch.as_tensor(b, dtype=torch.float64).flatten()
    den = b.norm().item()
    num = (a - b).norm().item()
    return num / den if den > 0 else num
