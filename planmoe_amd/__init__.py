"""planmoe_amd -- MI355X-native implementation of PlanMoE's per-GPU MoE data path."""
