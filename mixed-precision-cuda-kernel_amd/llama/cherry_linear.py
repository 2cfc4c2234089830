"""Training-time / fake-quant CherryQ linear.

Same surface as the reference's llama/cherry_linear.py: an `nn.Linear` whose weight is fake
quantised group-wise on the fly, except for the `cherry_indices` input channels, which stay in
full precision.  It is what `llama.qlinear.QuantLinear.pack()` consumes.  For fp16 and fp32
weights on a GPU the fake quantisation is one fused kernel of the HIP library (bit-identical to
the torch operations it replaces); other dtypes, layer-wise scales and CPU tensors go through
the torch operations.
"""
import math

import torch
import torch.nn as nn

from .quantizer import FullSymQuantizer, RestrictedSymQuantizer


class _FakeQuantSTE(torch.autograd.Function):
    """Fused fake quantisation in the straight-through form  (q - w) + w  of
    llama/cherry_linear.py:97-98: the forward value is that expression evaluated in the weight
    dtype, the gradient with respect to the weight is the incoming gradient."""

    @staticmethod
    def forward(ctx, weight, cherry_indices, w_bits, group_size):
        import quant_cuda
        return quant_cuda.fake_quant_cherryq(w_bits, weight.detach().contiguous(), cherry_indices, group_size,
                                             ste=True)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None, None


class _FakeQuantPlain(torch.autograd.Function):
    """Group-wise fake quantisation of the whole weight (no cherry channels) for the plain QAT
    branch: the value of FullSymQuantizer.forward without clipping (llama/quantizer.py:172-184),
    whose backward hands the gradient through unchanged (:120-133)."""

    @staticmethod
    def forward(ctx, weight, w_bits, group_size):
        import quant_cuda
        return quant_cuda.fake_quant_cherryq(w_bits, weight.detach().contiguous(), None, group_size, ste=False)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None


class QuantLinear(nn.Linear):
    def __init__(self, *args, bias=False, w_bits=16, weight_layerwise=False, group_size=-1,
                 cherryq=False, cherry_fraction=1 / 256):
        super().__init__(*args, bias=bias)
        self.w_bits = w_bits
        self.weight_layerwise = weight_layerwise
        self.group_size = group_size
        self.cherryq = cherryq
        self.cherry_fraction = cherry_fraction
        if 1 < self.w_bits < 16:
            if self.cherryq:
                # llama/cherry_linear.py:33: a multiple of 8 so that the packed rows stay whole
                self.num_cherries = math.ceil(self.weight.shape[-1] * cherry_fraction) // 8 * 8
                self.register_buffer("cherry_indices", -torch.ones(self.num_cherries, dtype=torch.int32))
                self.cherry_indices_registered = False
            self.quantizer = RestrictedSymQuantizer if self.w_bits > 4 else FullSymQuantizer
            self.dequantized = False

    def init_weights_(self):
        pass

    # ---- scales ---------------------------------------------------------------------------
    def _expand_scaling_factors(self, s, weight):
        if s.ndimension() == 0 or s.shape[-1] == 1:
            return s.expand_as(weight)
        return s.repeat_interleave(self.group_size, dim=-1)[:, :weight.shape[-1]]

    def _get_scaling_factors(self, weight):
        """(out, num_group) scales, groups of `group_size` consecutive columns of `weight`
        (the last may be short).  llama/cherry_linear.py:69-75."""
        step = self.group_size if self.group_size > 0 else weight.shape[-1]
        parts = [
            self.quantizer.get_scaling_factor(weight[:, i:i + step], None, self.w_bits, self.weight_layerwise)
            for i in range(0, weight.shape[-1], step)
        ]
        return torch.cat(parts, dim=-1)

    # ---- cherry channels --------------------------------------------------------------------
    def register_cherry_indices(self, cherry_indices):
        assert cherry_indices.shape[-1] >= self.cherry_indices.shape[-1], "The passed indices are invalid."
        self.cherry_indices = cherry_indices.to(dtype=torch.int32, device=self.weight.device)
        self.cherry_indices_registered = True

    def _normal_columns(self, width, device):
        keep = torch.ones(width, dtype=torch.bool, device=device)
        keep[self.cherry_indices.long()] = False
        return keep.nonzero().squeeze(1)

    def _fused_fake_quant(self, weight) -> bool:
        """Whether the HIP kernel computes this weight's fake quantisation: GPU tensor, fp16 or
        fp32, per-row group scales of the full-range quantiser, registered channels."""
        if not weight.is_cuda or self.quantizer is not FullSymQuantizer or self.weight_layerwise:
            return False
        if not getattr(self, "cherry_indices_registered", False):
            return False  # the torch operations raise on the placeholder indices, as the reference does
        import quant_cuda
        return quant_cuda.fake_quant_supported(weight, self.w_bits, self.group_size)

    def _fused_plain(self, weight) -> bool:
        """The same for the branch without cherry channels (groups must tile the row, as the
        reference's reshape demands)."""
        if not weight.is_cuda or self.quantizer is not FullSymQuantizer or self.weight_layerwise:
            return False
        if self.group_size <= 0 or weight.shape[1] % self.group_size:
            return False
        import quant_cuda
        return quant_cuda.fake_quant_supported(weight, self.w_bits, self.group_size)

    def _adjust_weight(self, weight: torch.Tensor, ste=True):
        """Weight with every non-cherry column fake quantised (groups run over the compacted
        normal columns); with `ste` the result carries the straight-through gradient.
        No clipping is applied (llama/cherry_linear.py:77-99)."""
        assert not self.training or self.cherry_indices_registered, "`cherry_indices` is not registered yet."
        if self._fused_fake_quant(weight):
            if ste:
                return _FakeQuantSTE.apply(weight, self.cherry_indices, self.w_bits, self.group_size)
            import quant_cuda
            return quant_cuda.fake_quant_cherryq(self.w_bits, weight.detach().contiguous(), self.cherry_indices,
                                                 self.group_size, ste=False)
        cols = self._normal_columns(weight.shape[1], weight.device)
        normal = weight.detach().index_select(-1, cols)
        s = self._expand_scaling_factors(self._get_scaling_factors(normal), normal)
        real_weight = weight.detach().clone()
        real_weight[..., cols] = self.quantizer.transform(normal, s, self.w_bits)
        if ste:
            real_weight = real_weight - weight.detach() + weight
        return real_weight

    @torch.inference_mode()
    def prepare_weight_for_inference(self, weight):
        """Replace `self.weight` by its fake-quantised value once (llama/cherry_linear.py:48-61)."""
        assert not self.training and not self.dequantized, \
            "Prepare during training or prepare an already dequantized model is not allowed."
        assert not self.cherryq or (self.cherry_indices >= 0).all(), "`cherry_indices` is invalid."
        if self.cherryq:
            self.weight.data.copy_(self._adjust_weight(weight, ste=False))
        else:
            grouped = weight.reshape(weight.shape[0], -1, self.group_size)
            s = self.quantizer.get_scaling_factor(grouped, None, self.w_bits, self.weight_layerwise)
            self.weight.data.copy_(self.quantizer.transform(grouped, s, self.w_bits).flatten(1))
        self.dequantized = True
        return self.weight

    # ---- forward ------------------------------------------------------------------------------
    def quant_forward(self, input_):
        assert self.weight.ndimension() == 2
        if self.w_bits >= 16:
            weight = self.weight
        elif self.w_bits > 1:
            weight = self.weight
            if self.cherryq:
                if self.training:
                    weight = self._adjust_weight(weight)
                elif not self.dequantized:
                    weight = self.prepare_weight_for_inference(weight)
            elif self.training and self._fused_plain(weight):
                weight = _FakeQuantPlain.apply(weight, self.w_bits, self.group_size)
            elif self.training:
                # plain QAT: group-wise fake quantisation through the autograd function
                grouped = weight.reshape(weight.shape[0], -1, self.group_size)
                s = self.quantizer.get_scaling_factor(grouped, None, self.w_bits, self.weight_layerwise)
                weight = self.quantizer.apply(grouped, None, self.w_bits, self.weight_layerwise, s).flatten(1)
            elif not self.dequantized:
                weight = self.prepare_weight_for_inference(weight)
        else:
            raise NotImplementedError(f"Quantization for {self.w_bits}bit is not implemented yet.")
        out = nn.functional.linear(input_, weight)
        if self.bias is not None:
            out += self.bias
        return out

    def forward(self, x: torch.Tensor, **kwargs) -> torch.Tensor:
        return self.quant_forward(x, **kwargs)
