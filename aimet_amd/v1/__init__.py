"""v1 (static-grid, DlQuantization arithmetic) quantization simulation: tensor quantizers, wrappers, QuantizationSimModel,
AdaRound."""
