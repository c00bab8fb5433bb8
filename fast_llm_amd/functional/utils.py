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


class _ForwardBackwardPair(torch.autograd.Function):
    """One autograd node for every wrapped pair: the pair itself travels as the first argument. The last argument is
    an empty tensor that requires a gradient, so that autograd visits the node even when none of the caller's tensors
    does (the weight gradients that `backward` writes are side effects autograd knows nothing about)."""

    @staticmethod
    def forward(ctx, pair: tuple[typing.Callable, typing.Callable], *arguments_and_anchor):
        run_forward, ctx.run_backward = pair
        *results, ctx.saved = _as_tuple(run_forward(*arguments_and_anchor[:-1]), "forward")
        ctx.num_inputs = len(arguments_and_anchor)
        return results[0] if len(results) == 1 else tuple(results)

    @staticmethod
    def backward(ctx, *grad_outputs):
        grads = ctx.run_backward(*grad_outputs, ctx.saved)
        if grads is None or isinstance(grads, torch.Tensor):
            grads = (grads,)
        # Gradients for the leading arguments, in order; none for the pair, the other arguments and the anchor.
        return (None, *grads) + (None,) * (ctx.num_inputs - len(grads))


def _as_tuple(value, what: str) -> tuple:
    if not isinstance(value, tuple) or not value:
        raise AssertionError(f"`{what}` must return a tuple that ends with its context, got {type(value).__name__}")
    return value


def wrap_forward_backward(
    forward: typing.Callable[..., tuple], backward: typing.Callable[..., typing.Any]
) -> typing.Callable[..., typing.Any]:
    """
    Wrap a (`forward`, `backward`) pair into a differentiable function.
    * `forward(input_, *args) -> (*outputs, context)`
    * `backward(*grad_outputs, context) -> grads of the leading arguments` (a tensor or a tuple).
    Keyword arguments are passed on positionally, in the order the caller wrote them (the reference's convention,
    fast_llm/functional/utils.py:52-54: the caller's keyword order must match `forward`'s positional order).
    """
    anchor = torch.empty(0, requires_grad=True)
    pair = (forward, backward)

    def differentiable(*args, **kwargs):
        return _ForwardBackwardPair.apply(pair, *args, *kwargs.values(), anchor)

    return differentiable


class AuxiliaryLoss(torch.autograd.Function):
    """`AuxiliaryLoss.apply(input_, aux_loss, grad)` is `input_`; back-propagating through it also sends the constant
    `grad` (None: nothing) into `aux_loss`, which trains on a loss that is attached at the tensor it regularises
    instead of being added to the objective. Reference: fast_llm/functional/utils.py:63-71."""

    @staticmethod
    def forward(ctx, input_: torch.Tensor, aux_loss: torch.Tensor, grad: float | None) -> torch.Tensor:
        ctx.loss_shape = (aux_loss.shape, aux_loss.dtype, aux_loss.device)
        ctx.loss_grad = grad
        return input_

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        loss_grad = None
        if ctx.loss_grad is not None:
            shape, dtype, device = ctx.loss_shape
            loss_grad = torch.full(shape, ctx.loss_grad, dtype=dtype, device=device)
        return grad_output, loss_grad, None
