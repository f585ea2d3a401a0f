"""mflux_amd -- MI355X-native group-wise affine quantization and quantized
linears, a drop-in for the MLX operations mflux's diffusion transformers run
through (``mx.quantize`` / ``nn.quantize`` / ``QuantizedLinear`` /
``mx.quantized_matmul``)."""
from . import lora, nn, weights
from .core import (PreparedWeights, dequantize, dequantize_rows, gelu_approx, layer_norm_modulate, prepare_weights, quantize,
                   quantized_matmul,
                   quantized_matmul_epilogue, quantized_matmul_prepared, silu, silu_quantized_matmul)

__all__ = ["nn", "lora", "weights", "quantize", "dequantize", "dequantize_rows", "quantized_matmul",
           "quantized_matmul_epilogue", "silu", "gelu_approx", "silu_quantized_matmul", "layer_norm_modulate",
           "prepare_weights", "quantized_matmul_prepared", "PreparedWeights"]
__version__ = "0.1.0"
