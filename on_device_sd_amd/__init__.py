"""MI355X-native MoE block (router -> top-k -> dispatch -> W4A16 SwiGLU experts -> combine).

Host code is Python on PyTorch-ROCm; all computation runs in hand-written gfx950 kernels
behind the C ABI of ``include/odsd_moe.h`` (``libodsd_moe.so`` next to this file).
"""
from .core import (AttentionOutput, ExpertID, ExpertPlacement, LayerOutput, MoEConfig,
                   RoutingResult)
from . import _lib, ops, workloads
from .w4 import W4ExpertBank, W4ExpertParams, build_table
from .runner import (MoEOnlyStack, W4MoERunner, expert_forward_with_weights, moe_layer_forward)
from .placement import (ExpertActivation, LayerExpertActivations, build_draft_placement,
                        build_layer_activations, build_prefill_placement)
from .layers import W4MoELayer, W4MoELayerWithWeights, W4Operators
from .cache import LRUStrategy, W4ExpertCache, cache_capacity
from .kv import (SequenceSlots, attention_for_context, build_decode_context, build_prefill_context,
                 build_verify_context, get_attention_context, paged_attention, store_kvcache, varlen_attention)

__all__ = [
    "AttentionOutput", "ExpertID", "ExpertPlacement", "LayerOutput", "MoEConfig", "RoutingResult",
    "W4ExpertBank", "W4ExpertParams", "build_table", "MoEOnlyStack", "W4MoERunner",
    "expert_forward_with_weights", "moe_layer_forward", "ops", "workloads",
    "ExpertActivation", "LayerExpertActivations", "build_layer_activations", "build_prefill_placement",
    "build_draft_placement",
    "W4MoELayer", "W4MoELayerWithWeights", "W4Operators",
    "LRUStrategy", "W4ExpertCache", "cache_capacity",
    "SequenceSlots", "build_verify_context", "build_prefill_context", "build_decode_context",
    "get_attention_context", "attention_for_context", "paged_attention", "store_kvcache", "varlen_attention",
]
