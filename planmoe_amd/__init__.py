"""planmoe_amd -- MI355X-native implementation of PlanMoE's per-GPU MoE data path.

Exports the names of the reference's ``moe.py`` (moe.py:6-12)."""
# Low-level ops
from .gating import fast_cumsum_sub_one
from .fast_dispatch import fast_dispatcher, extract_critical, fast_encode, fast_decode

top_k_routing = extract_critical

# High-level ops
from .moe_layer import moe_layer

__all__ = ["fast_cumsum_sub_one", "fast_dispatcher", "extract_critical", "top_k_routing",
           "fast_encode", "fast_decode", "moe_layer"]
