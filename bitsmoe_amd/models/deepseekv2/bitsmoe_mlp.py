from bitsmoe_amd.models.base_mlp import BitsMoE_BaseMoeMLP


class BitsMoE_DeepSeekMLP(BitsMoE_BaseMoeMLP):
    """Packed expert container of a DeepSeek-V2 layer (reference: bitsmoe/models/deepseekv2/bitsmoe_mlp.py)."""
