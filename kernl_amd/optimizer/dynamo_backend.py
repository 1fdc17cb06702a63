"""The ordered rewrite pipeline applied to every graph TorchDynamo captures
(reference: src/kernl/optimizer/dynamo_backend.py:25-34)."""
import torch

from kernl_amd.optimizer.attention import (
    fuse_attention_pattern_1,
    fuse_attention_pattern_2,
    fuse_attention_pattern_3,
    fuse_attention_scaled,
    fuse_attention_sdpa,
    share_mask_conversion,
)
from kernl_amd.optimizer.dropout import remove_dropout
from kernl_amd.optimizer.kv_cache import drop_empty_cat_operands
from kernl_amd.optimizer.layer_norm import (
    fuse_embeddings_into_layer_norm,
    replace_layer_norm,
    replace_layer_norm_fn,
    replace_layer_norm_rms,
)
from kernl_amd.optimizer.linear import (
    fuse_linears_into_add_layer_norms,
    fuse_residual_into_linears,
    fuse_rms_norm_into_linears,
    fuse_rms_stats_into_residual_adds,
    fuse_rotary_into_projections,
    replace_all_linear,
)
from kernl_amd.optimizer.mask import (
    constant_causal_masks_to_flag,
    drop_all_true_conjuncts,
    full_range_index_to_view,
    merge_nested_expands,
    scalar_tensors_to_full,
    sink_expand_below_where,
)
from kernl_amd.optimizer.normalizer import normalize_operators
from kernl_amd.optimizer.rotary import fuse_rotary_embedding


def dynamo_backend_ofi(gm: torch.fx.GraphModule, assume_causal=False):
    normalize_operators(gm)
    remove_dropout(gm)
    drop_empty_cat_operands(gm)
    fuse_rotary_embedding(gm)
    scalar_tensors_to_full(gm)
    drop_all_true_conjuncts(gm)
    full_range_index_to_view(gm)
    merge_nested_expands(gm)
    sink_expand_below_where(gm)
    merge_nested_expands(gm)
    fuse_attention_pattern_1(gm, assume_causal)
    fuse_attention_pattern_2(gm, assume_causal)
    fuse_attention_pattern_3(gm, assume_causal)
    fuse_attention_scaled(gm, assume_causal)
    fuse_attention_sdpa(gm, assume_causal)
    constant_causal_masks_to_flag(gm)
    share_mask_conversion(gm)
    replace_all_linear(gm)
    replace_layer_norm(gm)
    replace_layer_norm_fn(gm)
    replace_layer_norm_rms(gm)
    fuse_embeddings_into_layer_norm(gm)
    fuse_rms_norm_into_linears(gm)
    fuse_rotary_into_projections(gm)
    fuse_residual_into_linears(gm)
    fuse_linears_into_add_layer_norms(gm)
    fuse_rms_stats_into_residual_adds(gm)
    return gm
