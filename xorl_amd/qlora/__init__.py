"""Drop-in counterparts of ``xorl.qlora.modules`` backed by the HIP kernels."""

from .linear import (
    BlockFP8QLoRALinear,
    Int4QLoRALinear,
    LoraModule,
    NF4QLoRALinear,
    NvFP4QLoRALinear,
    QLoRALinear,
    deregister_qlora_weights_from_fsdp,
)

__all__ = [
    "LoraModule",
    "QLoRALinear",
    "BlockFP8QLoRALinear",
    "NvFP4QLoRALinear",
    "Int4QLoRALinear",
    "NF4QLoRALinear",
    "deregister_qlora_weights_from_fsdp",
]

from .moe_experts import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts, QLoRAMoeExperts  # noqa: E402

__all__ += ["QLoRAMoeExperts", "BlockFP8QLoRAMoeExperts", "NvFP4QLoRAMoeExperts", "NF4QLoRAMoeExperts"]

from .utils import maybe_load_prequantized_qlora, maybe_requant_qlora  # noqa: E402

__all__ += ["maybe_load_prequantized_qlora", "maybe_requant_qlora"]

from .inline_buffers import (  # noqa: E402
    BlockFP8QLoRAExpertBuffer,
    BlockFP8WeightBuffer,
    NvFP4QLoRAExpertBuffer,
    NvFP4WeightBuffer,
    QLoRAExpertBuffer,
    QLoRAWeightBuffer,
    parse_expert_full_key,
)

__all__ += ["QLoRAWeightBuffer", "NvFP4WeightBuffer", "BlockFP8WeightBuffer", "QLoRAExpertBuffer",
            "NvFP4QLoRAExpertBuffer", "BlockFP8QLoRAExpertBuffer", "parse_expert_full_key"]
