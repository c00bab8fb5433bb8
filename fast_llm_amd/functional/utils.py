"""
Autograd glue and argument checks (reference: fast_llm/functional/utils.py:13-56, fast_llm/utils.py:35-42,84-200).
"""

import typing

import torch


class Assert:
    """The subset of the reference's `Assert` helpers that the hot path uses; failures are `AssertionError`s."""

    @staticmethod
    def eq(x, *args, msg=None):
        for arg in args:
            assert x == arg, f"{x} != {arg}" + ("" if msg is None else f" | {msg}")

    @staticmethod
    def custom(fn, *args, **kwargs):
        assert fn(*args, **kwargs), f"Assertion failed: fn({', '.join(map(str, args))})"


def div(x: int, y: int) -> int:
    """Exact division; `ValueError` when `y` does not divide `x`."""
    if x % y != 0:
        raise ValueError(f"{x}%{y}!=0")
    return x // y


def wrap_forward_backward(
    forward: typing.Callable[..., tuple], backward: typing.Callable[..., typing.Any]
) -> typing.Callable[..., typing.Any]:
    """
    Wrap a (`forward`, `backward`) pair into a differentiable function.
    * `forward(input_, *args) -> (*outputs, context)`
    * `backward(*grad_outputs, context) -> grads of the leading arguments` (a tensor or a tuple).
    Keyword arguments are passed on positionally in the order given, as the reference does.
    """

    # Backward must run even if no input requires a gradient (weight gradients are side effects).
    in_ = torch.empty(0, requires_grad=True)

    class Function(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *args):
            outputs = forward(*args[:-1])
            Assert.custom(isinstance, outputs, tuple)
            ctx.context = outputs[-1]
            ctx.nargs = len(args)
            if len(outputs) == 2:
                return outputs[0]
            return outputs[:-1]

        @staticmethod
        def backward(ctx, *grad_outputs):
            grad_input = backward(*grad_outputs, ctx.context)
            if not isinstance(grad_input, tuple):
                assert isinstance(grad_input, torch.Tensor) or grad_input is None
                grad_input = (grad_input,)
            return (*grad_input, *[None for _ in range(ctx.nargs - len(grad_input))])

    def call(*args, **kwargs):
        return Function.apply(*args, *kwargs.values(), in_)

    return call


class AuxiliaryLoss(torch.autograd.Function):
    """Identity on `input_` whose backward also hands the constant `grad` to `aux_loss`: attaches an auxiliary loss
    to the graph at the tensor it regularises. Reference: fast_llm/functional/utils.py:63-71."""

    @staticmethod
    def forward(ctx, input_: torch.Tensor, aux_loss: torch.Tensor, grad: float | None) -> torch.Tensor:  # noqa
        ctx.grad = None if grad is None else torch.full_like(aux_loss, grad)
        return input_

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> tuple[torch.Tensor | None, ...]:  # noqa
        return grad_output, ctx.grad, None
