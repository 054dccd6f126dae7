"""flexsae_amd: the fused SAE decoder-loss path (TopK / HierarchicalTopK, forward + backward)
as hand-written HIP kernels for AMD MI355X (gfx950), behind the reference package's names.

    import flexsae_amd as flex
    loss = flex.triton_hierarchical_sae_loss(indices, weight, vals, bias, target)
    loss.backward()

Public names mirror reference torch-ext/flex_sae/__init__.py:5-18.  The ``triton_*`` names are
kept so that existing callers need no edit; nothing here uses Triton.
"""
from .ops import (check_index_flag, hier_stage_bytes, hierarchical_sae_sgd_step, set_dense_latents,
                  set_fused_training,
                  set_hier_min_slice_cols, set_hier_scratch_bytes, set_hier_stage_bytes, set_hot_latents,
                  set_index_checking, set_topk_residual_bf16, shared_pair_list, triton_hierarchical_sae_loss,
                  triton_topk_sae_loss)
from .reference import hierarchical_sae_loss, topk_sae_loss

# spelled-out aliases for new code
fused_hierarchical_sae_loss = triton_hierarchical_sae_loss
fused_topk_sae_loss = triton_topk_sae_loss

__kernel_metadata__ = {
    "license": "Apache-2.0",
    "backend": "hip",
    "arch": "gfx950",
}

__all__ = [
    "__kernel_metadata__",
    "topk_sae_loss",
    "triton_topk_sae_loss",
    "hierarchical_sae_loss",
    "triton_hierarchical_sae_loss",
    "fused_topk_sae_loss",
    "fused_hierarchical_sae_loss",
    "hierarchical_sae_sgd_step",
    "check_index_flag",
    "set_index_checking",
    "set_hier_scratch_bytes",
    "set_hier_min_slice_cols",
    "set_hier_stage_bytes",
    "hier_stage_bytes",
    "set_fused_training",
    "set_hot_latents",
    "set_dense_latents",
    "set_topk_residual_bf16",
    "shared_pair_list",
]
