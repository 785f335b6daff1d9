"""Helpers of the path with the reference's names (asdl/utils.py)."""
from contextlib import contextmanager

import torch
from torch import nn

from . import kernels
from .profiling import nvtx_range

_REQUIRES_GRAD_ATTR = '_original_requires_grad'

__all__ = ['original_requires_grad', 'record_original_requires_grad', 'restore_original_requires_grad',
           'skip_param_grad', 'cholesky_inv', 'has_reduction', 'nvtx_range', 'UnfoldedInput', 'im2col_2d']


def original_requires_grad(module=None, param_name=None, param=None):
    """asdl/utils.py:21-27."""
    if param is None:
        if module is None or param_name is None:
            raise ValueError('Both module and param_name have to be set.')
        param = getattr(module, param_name, None)
    return param is not None and getattr(param, _REQUIRES_GRAD_ATTR)


def record_original_requires_grad(param):
    setattr(param, _REQUIRES_GRAD_ATTR, param.requires_grad)


def restore_original_requires_grad(param):
    param.requires_grad = getattr(param, _REQUIRES_GRAD_ATTR, param.requires_grad)


@contextmanager
def skip_param_grad(model, disable=False):
    """Parameters stop accumulating .grad while the Fisher backward runs (asdl/utils.py:38-48)."""
    if not disable:
        for param in model.parameters():
            record_original_requires_grad(param)
            param.requires_grad = False
    yield
    if not disable:
        for param in model.parameters():
            restore_original_requires_grad(param)


def cholesky_inv(X, damping=1e-7):
    """(X + damping I)^-1 on the GPU; X is left unchanged; raises torch.linalg.LinAlgError when
    the damped matrix is not positive definite (asdl/utils.py:91-96)."""
    return kernels.cholesky_inv(X, float(damping))


def has_reduction(func):
    """asdl/utils.py:197-204."""
    if isinstance(func, nn.Module):
        return hasattr(func, 'reduction')
    elif callable(func):
        return 'reduction' in func.__code__.co_varnames
    return False


class UnfoldedInput:
    """Stands for the unfolded patches [n, c*kh*kw, h_out*w_out] of a Conv2d input without
    building them: the factor kernel reads the NCHW tensor and applies the unfold on the fly."""

    def __init__(self, x, kernel_size, stride, padding):
        self.x = x
        self.kernel_size = tuple(kernel_size)
        self.stride = tuple(stride)
        self.padding = tuple(padding)
        n, c, h, w = x.shape
        self.h_out = (h + 2 * self.padding[0] - self.kernel_size[0]) // self.stride[0] + 1
        self.w_out = (w + 2 * self.padding[1] - self.kernel_size[1]) // self.stride[1] + 1

    @property
    def shape(self):
        n, c = self.x.shape[:2]
        return (n, c * self.kernel_size[0] * self.kernel_size[1], self.h_out * self.w_out)

    @property
    def out_size(self):
        return self.h_out * self.w_out


def im2col_2d(x, conv2d):
    """Same argument checks as asdl/utils.py:51-59; returns the lazy UnfoldedInput."""
    if x.ndim != 4:
        raise ValueError(f'x.ndim has to be 4. Got {x.ndim}.')
    if not isinstance(conv2d, (nn.Conv2d, nn.ConvTranspose2d)):
        raise TypeError(f'conv2d has to be {nn.Conv2d} or {nn.ConvTranspose2d}. Got {type(conv2d)}.')
    if conv2d.dilation != (1, 1):
        raise ValueError(f'conv2d.dilation has to be (1, 1). Got {conv2d.dilation}.')
    padding = conv2d.padding if conv2d.padding != 'valid' else (0, 0)
    if isinstance(padding, str):
        raise ValueError(f"conv2d.padding has to be a tuple or 'valid'. Got {padding}.")
    return UnfoldedInput(x, conv2d.kernel_size, conv2d.stride, padding)
