"""
The gradient-buffer convention of parameters on the hot path (reference: fast_llm/tensor.py:345-355).

A weight carries `grad_buffer` (the tensor its gradient is written into) and `param_grad_is_zero` (True until the first
write of the current accumulation window). The first write overwrites, later ones accumulate.
"""

import torch


def param_get_and_unset_is_zero(param: torch.Tensor) -> bool:
    is_zero = param.param_grad_is_zero
    param.param_grad_is_zero = False
    return is_zero


def accumulate_gradient(param: torch.Tensor, grad: torch.Tensor) -> None:
    if param_get_and_unset_is_zero(param):
        param.grad_buffer.copy_(grad)
    else:
        param.grad_buffer.add_(grad)
