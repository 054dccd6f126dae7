"""Pure-torch definitions of the two losses (device-agnostic, autograd by torch).

These are the public ``topk_sae_loss`` / ``hierarchical_sae_loss`` names of the reference
package (reference torch-ext/flex_sae/__init__.py:12-18; definitions at
torch-ext/flex_sae/topk_kernels.py:226-237 and torch-ext/flex_sae/hierarchical_kernels.py:312-323):
slow, memory-hungry (they materialise ``[B,K,D]``), kept because callers use them as the
eager baseline next to the fused ops.  The fused ops never route through them.
"""
import torch


def _gathered(indices: torch.Tensor, weight: torch.Tensor, vals: torch.Tensor) -> torch.Tensor:
    # [B,K,D] fp32: each selected decoder row scaled by its activation
    return weight[indices].to(torch.float32) * vals.unsqueeze(-1)


def topk_sae_loss(indices: torch.Tensor, weight: torch.Tensor, vals: torch.Tensor,
                  bias: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    """mean over (B,D) of (bias + sum_k vals*W[idx] - target)^2, computed in fp32."""
    recon = bias.to(torch.float32) + _gathered(indices, weight, vals).sum(dim=1)
    return (recon.to(torch.float32) - target.to(torch.float32)).pow(2).mean()


def hierarchical_sae_loss(indices: torch.Tensor, weight: torch.Tensor, vals: torch.Tensor,
                          bias: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    """mean over (B,K,D) of (bias + prefix-sum_k vals*W[idx] - target)^2, computed in fp32."""
    recon = bias.to(torch.float32) + _gathered(indices, weight, vals).cumsum(dim=1)
    return (recon.to(torch.float32) - target.to(torch.float32).unsqueeze(1)).pow(2).mean()
