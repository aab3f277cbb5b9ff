"""Backend registry of the v2 affine quantization functions
(TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/utils.py:45-104).

A backend is any module-like object with quantize / dequantize / quantize_dequantize of the protocol below.  The
backend registered here by default is ``hip_gfx950`` (hand-written HIP kernels); there is no torch-ops backend."""
from typing import List, Optional, Protocol

import torch

from ....utils import _ContextManager
from . import hip_gfx950


class _QuantizationBackendProtocol(Protocol):
    def quantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
                 block_size: Optional[List] = None) -> torch.Tensor: ...

    def dequantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
                   block_size: Optional[List] = None) -> torch.Tensor: ...

    def quantize_dequantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int,
                            qmax: int, block_size: Optional[List] = None) -> torch.Tensor: ...


_CURRENT_BACKEND = 'hip_gfx950'
_SUPPORTED_BACKENDS = {'hip_gfx950': hip_gfx950}


def set_global_backend(name: str):
    global _CURRENT_BACKEND  # pylint: disable=global-statement
    if name not in _SUPPORTED_BACKENDS:
        raise RuntimeError(f"Backend '{name}' is not supported. Please choose one of: "
                           f"{', '.join(_SUPPORTED_BACKENDS)}")
    _CURRENT_BACKEND = name


def set_backend(name: str) -> _ContextManager:
    if name not in _SUPPORTED_BACKENDS:
        raise RuntimeError(f"Backend '{name}' is not supported. Please choose one of: "
                           f"{', '.join(_SUPPORTED_BACKENDS)}")
    old_backend = _CURRENT_BACKEND
    return _ContextManager(action=lambda: set_global_backend(name), cleanup=lambda: set_global_backend(old_backend))


def get_backend() -> _QuantizationBackendProtocol:
    return _SUPPORTED_BACKENDS[_CURRENT_BACKEND]


def add_backend(name: str, module: _QuantizationBackendProtocol):
    if name in _SUPPORTED_BACKENDS:
        raise RuntimeError(f'{name} is exist.')
    _SUPPORTED_BACKENDS[name] = module


__all__ = ['set_global_backend', 'set_backend', 'get_backend', 'add_backend']
