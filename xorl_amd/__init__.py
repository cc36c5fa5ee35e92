"""xorl_amd: MI355X-native QLoRA quantized-linear path (drop-in for xorl's QLoRA modules)."""

__version__ = "0.1.0"
