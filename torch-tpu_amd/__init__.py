"""MI355X-native FP8 fused-MoE inference path behind torch-tpu's `my_ops` operator surface.

Importing the package loads libmoe_hip.so (hand-written gfx950 kernels behind a C ABI) and
registers `torch.ops.my_ops.{fused_moe_fused_experts, fused_moe_fused_experts_v2, noaux_tc_topk,
fused_moe_grouped_topk, mlp_w8a16_dq_forward, mm_w8a16_dq_forward, mlp_w8a8_quant_forward, moe_route, moe_permute, moe_pack_weights}`.  There is no CPU fallback: without the built library the import fails.
"""
from . import _lib                      # noqa: F401  (raises if the library is missing)
from . import my_ops as _my_ops         # noqa: F401  (registers torch.ops.my_ops.*)
from .my_ops import invalidate_weight_cache, set_expert_numerics
from .layer import FusedMoE, FusedMoEModule, convert_hf_moe_layer, pack_expert_weights, quant_weight_block128, stack_expert_weights, synthetic_weights
from .ops import (MoeHipError, act_quant, layer_eligible, layer_fp8, layer_workspace_bytes,
                  fused_experts_bf16, fused_experts_fp8, fused_experts_w8a16, fused_experts_workspace_bytes, gemm1_swiglu, gemm2, mlp_fp8, mm_bf16, mm_fp8, mm_w8a16,
                  moe_permute, moe_route, noaux_tc_topk, pack_layer, pack_weights, router_logits, scale_pitch, set_shared_overlap, tile_rows,
                  unpack_weights, weighted_reduce)

__all__ = ["FusedMoE", "FusedMoEModule", "set_expert_numerics", "invalidate_weight_cache", "convert_hf_moe_layer", "pack_expert_weights", "quant_weight_block128", "MoeHipError", "act_quant",
           "layer_eligible", "layer_fp8", "layer_workspace_bytes", "fused_experts_bf16", "fused_experts_fp8", "fused_experts_w8a16",
           "fused_experts_workspace_bytes", "gemm1_swiglu", "gemm2", "mlp_fp8", "mm_bf16", "mm_fp8", "mm_w8a16", "moe_permute", "moe_route", "noaux_tc_topk", "router_logits",
           "scale_pitch", "set_shared_overlap", "tile_rows", "weighted_reduce", "pack_weights", "unpack_weights", "pack_layer", "stack_expert_weights", "synthetic_weights"]
