"""Quantiser arithmetic of CherryQ (host side, plain torch).

Same public surface as the reference's llama/quantizer.py: `iinfo`, `get_max_input`,
`Quantizer`, `FullSymQuantizer` (w_bits <= 4, half-integer grid, llama/quantizer.py:136-207)
and `RestrictedSymQuantizer` (5..15 bits, llama/quantizer.py:64-133).  Every function keeps the
reference's operation order and dtypes, because the packed bytes depend on them at rounding
ties: the quotient input / S is formed in the input dtype, `quantize` continues in float32,
`transform` stays in the input dtype.
"""
from collections import namedtuple
from typing import Optional

import torch

iinfo = namedtuple("iinfo", ["min", "max"])


def get_max_input(input, clip_val, layerwise):
    """max |input|: one scalar if `layerwise`, else per last-dim row (keepdim).
    llama/quantizer.py:10-34."""
    if clip_val is not None:
        input = input.clamp(clip_val[0], clip_val[1])
    if layerwise:
        return input.abs().max()
    if input.ndimension() <= 3:
        return input.abs().amax(dim=-1, keepdim=True).detach()
    if input.ndimension() == 4:
        flat = input.reshape(input.shape[0], input.shape[1], -1)
        return flat.abs().amax(dim=-1, keepdim=True).unsqueeze(-1).detach()
    raise ValueError(f"Not implemented for shape: {input.shape}")


class Quantizer:
    """Interface shared by the two symmetric quantisers."""

    @staticmethod
    def iinfo(num_bits) -> iinfo:
        raise NotImplementedError

    @staticmethod
    def get_scaling_factor(input, clip_val, num_bits, layerwise):
        raise NotImplementedError

    @staticmethod
    def quantize(input, S, num_bits):
        raise NotImplementedError

    @staticmethod
    def dequantize(rounded_input, S):
        raise NotImplementedError

    @staticmethod
    def transform(input, S, num_bits):
        raise NotImplementedError


def _ste_backward(ctx, grad_output):
    # straight-through: pass the gradient, zero it where the input was clipped
    input, clip_val = ctx.saved_tensors
    grad = grad_output.clone()
    if clip_val is not None:
        grad[input.ge(clip_val[1])] = 0
        grad[input.le(clip_val[0])] = 0
    return grad, None, None, None, None


class FullSymQuantizer(Quantizer, torch.autograd.Function):
    """Uniform symmetric grid using every code: integers q in [-2^(b-1), 2^(b-1) - 1] stand for
    the values (q + 0.5) * S."""

    @staticmethod
    def iinfo(num_bits):
        half = 2 ** (num_bits - 1)
        return iinfo(min=-half, max=half - 1)

    @staticmethod
    def get_scaling_factor(input, clip_val, num_bits, layerwise):
        return (get_max_input(input, clip_val, layerwise) + 1e-6) / (2 ** (num_bits - 1))

    @staticmethod
    def _grid(ratio, num_bits):
        qmax = 2 ** (num_bits - 1) - 1e-2
        return torch.round(ratio.clamp(-qmax, qmax) - 0.5)

    @staticmethod
    def quantize(input, S, num_bits):
        ratio = (input / S.expand_as(input)).float()
        return FullSymQuantizer._grid(ratio, num_bits).to(torch.int32)

    @staticmethod
    def dequantize(rounded_input, S):
        s = S.expand_as(rounded_input)
        return (rounded_input.to(s.dtype) + 0.5) * s

    @staticmethod
    def transform(input, S, num_bits):
        s = S.expand_as(input)
        return (FullSymQuantizer._grid(input / s, num_bits) + 0.5) * s

    @staticmethod
    def forward(ctx, input, clip_val, num_bits, layerwise, S: Optional[torch.Tensor] = None):
        ctx.save_for_backward(input, clip_val)
        if clip_val is not None:
            input = input.clamp(clip_val[0], clip_val[1])
        if S is None:
            S = FullSymQuantizer.get_scaling_factor(input, clip_val, num_bits, layerwise)
        return FullSymQuantizer.transform(input, S, num_bits)

    @staticmethod
    def backward(ctx, grad_output):
        return _ste_backward(ctx, grad_output)


class RestrictedSymQuantizer(Quantizer, torch.autograd.Function):
    """Uniform symmetric grid without the most negative code: q in [-(2^(b-1)-1), 2^(b-1)-1]
    stands for q * S."""

    @staticmethod
    def iinfo(num_bits):
        top = 2 ** (num_bits - 1) - 1
        return iinfo(min=-top, max=top)

    @staticmethod
    def get_scaling_factor(input, clip_val, num_bits, layerwise):
        return (get_max_input(input, clip_val, layerwise) + 1e-6) / (2 ** (num_bits - 1) - 1)

    @staticmethod
    def quantize(input, S, num_bits):
        top = 2 ** (num_bits - 1) - 1
        ratio = (input / S.expand_as(input)).float()
        return torch.round(ratio).clamp(-top, top).to(torch.int32)

    @staticmethod
    def dequantize(rounded_input, S):
        s = S.expand_as(rounded_input)
        return rounded_input.to(s.dtype) * s

    @staticmethod
    def transform(input, S, num_bits):
        top = 2 ** (num_bits - 1) - 1
        s = S.expand_as(input)
        return torch.round(input / s).clamp(-top, top) * s

    @staticmethod
    def forward(ctx, input, clip_val, num_bits, layerwise, S: Optional[torch.Tensor] = None):
        ctx.save_for_backward(input, clip_val)
        if clip_val is not None:
            input = input.clamp(clip_val[0], clip_val[1])
        if S is None:
            S = RestrictedSymQuantizer.get_scaling_factor(input, clip_val, num_bits, layerwise)
        s = S.expand_as(input)
        return torch.round(input / s) * s  # the reference's forward does not clamp (:115)

    @staticmethod
    def backward(ctx, grad_output):
        return _ste_backward(ctx, grad_output)
