"""MI355X-native fused 4-bit AdamW (drop-in for the reference's quantized AdamW step).

    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    opt = AdamWFused_QuantFour(model.parameters(), lr=1e-3, betas=(0.9, 0.999),
                               eps=1e-8, weight_decay=1e-2)

The step runs in csrc/libq4adamw.so (build: python -m quantfour_adamw_cuda_amd.build).
"""
from .fused_quantfour import AdamWFused_QuantFour, enable_param_quantization
from .quantfour_hip import (dequantize_state, fused_4bit, fused_4bit_multi, fused_single_tensor,
                            fused_single_tensor_multi, quantize_state, state_sizes)

__all__ = [
    "AdamWFused_QuantFour",
    "enable_param_quantization",
    "fused_4bit",
    "fused_4bit_multi",
    "fused_single_tensor",
    "fused_single_tensor_multi",
    "state_sizes",
    "quantize_state",
    "dequantize_state",
]
