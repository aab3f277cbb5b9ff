"""AdaRound for the v1 quantization-simulation path."""
