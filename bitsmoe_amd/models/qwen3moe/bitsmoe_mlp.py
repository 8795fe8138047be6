from bitsmoe_amd.models.base_mlp import BitsMoE_BaseMoeMLP


class BitsMoE_Qwen3MoeMLP(BitsMoE_BaseMoeMLP):
    """Packed expert container of a Qwen3-MoE layer (reference: bitsmoe/models/qwen3moe/bitsmoe_mlp.py)."""
