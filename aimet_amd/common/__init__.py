"""Framework-agnostic value types and constants (the subset of aimet_common the quantization-simulation path uses)."""
