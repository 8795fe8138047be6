from bitsmoe_amd.models.base_mlp import BitsMoE_BaseMoeMLP


class BitsMoE_Qwen3NextMLP(BitsMoE_BaseMoeMLP):
    """Packed expert container of a Qwen3-Next layer (reference: bitsmoe/models/qwen3next/bitsmoe_mlp.py)."""
