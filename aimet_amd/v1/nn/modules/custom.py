"""Module forms of functional ops, so that quantization wrappers can be attached to them
(the reference's aimet_torch/v1/nn/modules/custom.py:149 and neighbours; normally inserted by its model preparer)."""
import torch
from torch import nn


class Add(nn.Module):
    @staticmethod
    def forward(x, y):
        return x + y


class Subtract(nn.Module):
    @staticmethod
    def forward(x, y):
        return x - y


class Multiply(nn.Module):
    @staticmethod
    def forward(x, y):
        return x * y


class Concat(nn.Module):
    def __init__(self, axis: int = 0):
        super().__init__()
        self._axis = axis

    def forward(self, *x):
        return torch.cat(x, dim=self._axis)


class Divide(nn.Module):
    @staticmethod
    def forward(x, y):
        return x / y


class MatMul(nn.Module):
    @staticmethod
    def forward(x, y):
        return torch.matmul(x, y)


class Addmm(nn.Module):
    """beta * input + alpha * (mat1 @ mat2), with the scaling factors as keyword arguments."""

    @staticmethod
    def forward(input, mat1, mat2, **kwargs):  # pylint: disable=redefined-builtin
        return torch.addmm(input, mat1, mat2, **kwargs)
