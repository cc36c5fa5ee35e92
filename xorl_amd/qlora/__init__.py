"""Drop-in counterparts of ``xorl.qlora.modules`` backed by the HIP kernels."""

from .linear import (
    BlockFP8QLoRALinear,
    Int4QLoRALinear,
    LoraModule,
    NF4QLoRALinear,
    NvFP4QLoRALinear,
    QLoRALinear,
    deregister_qlora_weights_from_fsdp,
    qlora_gate_up_silu,
    qlora_linears_forward,
    qlora_mlp_forward,
)

__all__ = [
    "LoraModule",
    "QLoRALinear",
    "BlockFP8QLoRALinear",
    "NvFP4QLoRALinear",
    "Int4QLoRALinear",
    "NF4QLoRALinear",
    "deregister_qlora_weights_from_fsdp",
    "qlora_gate_up_silu",
    "qlora_linears_forward",
    "qlora_mlp_forward",
]

from .moe_experts import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts, QLoRAMoeExperts  # noqa: E402

__all__ += ["QLoRAMoeExperts", "BlockFP8QLoRAMoeExperts", "NvFP4QLoRAMoeExperts", "NF4QLoRAMoeExperts"]

from .utils import (  # noqa: E402
    detect_prequantized_block_fp8,
    detect_prequantized_nvfp4,
    inject_qlora_into_model,
    maybe_load_and_quantize_moe_qlora,
    maybe_load_prequantized_qlora,
    maybe_merge_lora,
    maybe_quantize_qlora,
    maybe_requant_qlora,
    reset_lora_optimizer_states,
    save_qlora_checkpoint,
)

__all__ += ["inject_qlora_into_model", "maybe_load_prequantized_qlora", "maybe_load_and_quantize_moe_qlora",
            "maybe_quantize_qlora", "maybe_requant_qlora", "save_qlora_checkpoint", "detect_prequantized_nvfp4",
            "detect_prequantized_block_fp8", "maybe_merge_lora", "reset_lora_optimizer_states"]

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
