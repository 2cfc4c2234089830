"""Inference-time CherryQ linear over packed buffers, MI355X build.

Same class surface and state-dict schema as the reference's llama/qlinear.py:13-199:

    cherry_indices (C,) int16 | cherry_weight (C, out) fp16 | qweight (Kn/8*w_bits, out) uint8
    scales (ceil(Kn/G), out) fp16 | bias (out,) fp16 or None

`forward` runs the fused HIP kernels through the `quant_cuda` entry points (fused mode) or, under
`QuantLinear.dmode(layerwise_dequantize=False)`, unpacks once to a dense fp16 weight and uses a
plain linear, exactly as the reference does.  `pack()` and `unpack()` are host logic in torch;
on GPU tensors `unpack()` uses the library's dequantisation kernel, which yields the same bits.
"""
import math
from contextlib import contextmanager

import torch
import torch.nn as nn

import quant_cuda

from .cherry_linear import QuantLinear as QuantLinearForTraining
from .quantizer import FullSymQuantizer, Quantizer


def pack_codes(codes: torch.Tensor, w_bits: int) -> torch.Tensor:
    """codes (Kn, out) uint8 in [0, 2^b) -> qweight (Kn/8*b, out) uint8.

    Layout of llama/qlinear.py:86-116: for b in {2,4,8} byte row r holds the 8/b consecutive
    codes starting at (8/b) r, lowest bits first; for b = 3 every 8 codes of a column form one
    little-endian 24-bit word stored in three consecutive byte rows."""
    kn, n = codes.shape
    c = codes.to(torch.int32)
    if w_bits in (2, 4, 8):
        per = 8 // w_bits
        q = torch.zeros((kn // per, n), dtype=torch.int32, device=codes.device)
        for t in range(per):
            q |= c[t::per] << (w_bits * t)
        return q.to(torch.uint8)
    if w_bits == 3:
        units = c.reshape(kn // 8, 8, n)
        word = torch.zeros((kn // 8, n), dtype=torch.int32, device=codes.device)
        for i in range(8):
            word |= units[:, i] << (3 * i)
        rows = torch.stack([(word >> (8 * j)) & 0xFF for j in range(3)], dim=1)
        return rows.reshape(kn // 8 * 3, n).to(torch.uint8)
    raise NotImplementedError(f"{w_bits} bit is not implemented yet.")


def unpack_codes(qweight: torch.Tensor, w_bits: int) -> torch.Tensor:
    """Inverse of pack_codes: (Kn/8*b, out) uint8 -> codes (Kn, out) uint8."""
    rows, n = qweight.shape
    q = qweight.to(torch.int32)
    if w_bits in (2, 4, 8):
        per = 8 // w_bits
        parts = [(q >> (w_bits * t)) & (2 ** w_bits - 1) for t in range(per)]
        return torch.stack(parts, dim=1).reshape(rows * per, n).to(torch.uint8)
    if w_bits == 3:
        q = q.reshape(rows // 3, 3, n)
        word = q[:, 0] | (q[:, 1] << 8) | (q[:, 2] << 16)
        parts = [(word >> (3 * i)) & 7 for i in range(8)]
        return torch.stack(parts, dim=1).reshape(rows // 3 * 8, n).to(torch.uint8)
    raise NotImplementedError(f"{w_bits} bit is not implemented yet.")


class QuantLinear(nn.Module):

    _layerwise_dequantize = True
    # Rows at and above which the fused forward dequantises once and calls the library's dense GEMM
    # instead of the fused dequantise + MFMA kernel (measured crossover on MI355X: the fused kernel
    # is 1.6x faster at 128 rows of a 4096 -> 11008 layer, level at 512, 1.3x slower at 2048).
    prefill_rows = 512
    @classmethod
    @contextmanager
    def dmode(cls, layerwise_dequantize=True):
        """True (default): fused kernels dequantise on the fly at every call.  False: the first
        call unpacks to a dense fp16 weight that later calls reuse.  llama/qlinear.py:17-23."""
        mode = cls._layerwise_dequantize
        cls._layerwise_dequantize = layerwise_dequantize
        try:
            yield
        finally:
            cls._layerwise_dequantize = mode

    def __init__(self, w_bits, group_size, quantizer: Quantizer, cherry_fraction: float,
                 in_features, out_features, bias=True, **kwargs):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.w_bits = w_bits
        self.group_size = group_size if group_size != -1 else in_features
        self.quantizer = quantizer
        self.cherry_fraction = cherry_fraction
        self.num_cherries = math.ceil(in_features * cherry_fraction) // 8 * 8
        self.num_normal = self.in_features - self.num_cherries

        assert in_features % 8 == 0
        assert out_features % 8 == 0

        self.register_buffer("cherry_indices", torch.zeros(self.num_cherries, dtype=torch.int16))
        self.register_buffer("cherry_weight",
                             torch.zeros((self.num_cherries, self.out_features), dtype=torch.float16))
        self.register_buffer("qweight",
                             torch.zeros((self.num_normal // 8 * self.w_bits, out_features), dtype=torch.uint8))
        self.register_buffer("scales",
                             torch.zeros((math.ceil(self.num_normal / self.group_size), out_features),
                                         dtype=torch.float16))
        # `bias` may arrive as a bool or, from make_quant (utils.py:81-84), as the old module's
        # bias tensor / None; a multi-element tensor has no truth value, so test it explicitly
        has_bias = bias is not None and not (isinstance(bias, bool) and not bias)
        if has_bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float16))
        else:
            self.bias = None
        self.dequantized = False
        # the repacked weight stream of prepack() (not part of the state dict) and whether the
        # checkpoint-layout buffers were released in its favour
        self._stream = None
        self._released = False

    # ---- packing (host logic) ---------------------------------------------------------------
    def _normal_columns(self, device):
        keep = torch.ones(self.in_features, dtype=torch.bool, device=device)
        keep[self.cherry_indices.long().to(device)] = False
        return keep.nonzero().squeeze(1)

    @torch.inference_mode()
    def pack(self, linear: QuantLinearForTraining):
        """Fill the packed buffers from a fake-quant training module.  llama/qlinear.py:67-118.
        The buffers end up on the CPU, as in the reference."""
        self._drop_stream()  # a stream made from the old buffers must not outlive them
        if linear.bias is not None:
            self.bias = linear.bias.detach().to(torch.float16).cpu().clone()
        weight = linear.weight
        if (weight.is_cuda and weight.dtype == torch.float16 and self.w_bits in (3, 4)
                and linear.quantizer is FullSymQuantizer):
            # same arithmetic on the device; the buffers stay on the weight's device
            if self.bias is not None:
                self.bias = self.bias.to(weight.device)
            group = linear.group_size if linear.group_size != -1 else weight.shape[1]
            (self.cherry_indices, self.cherry_weight, self.qweight,
             self.scales) = quant_cuda.pack_cherryq(self.w_bits, weight.detach().contiguous(),
                                                    linear.cherry_indices, group)
            return
        cherry = linear.cherry_indices.sort().values.long()
        self.cherry_indices = cherry.to(dtype=torch.int16).cpu()
        self.cherry_weight = weight.t()[cherry].to(torch.float16).cpu()
        keep = torch.ones(weight.shape[1], dtype=torch.bool, device=weight.device)
        keep[cherry] = False
        normal_weight = weight[..., keep.nonzero().squeeze(1)].reshape(weight.shape[0], -1)
        scales = linear._get_scaling_factors(normal_weight).to(torch.float16)  # (out, groups)
        self.scales = scales.t().contiguous().cpu()
        expanded = scales.repeat_interleave(linear.group_size, dim=1)[:, :normal_weight.shape[1]]
        q = linear.quantizer.quantize(normal_weight, expanded, linear.w_bits)
        codes = (q.t().contiguous() - linear.quantizer.iinfo(linear.w_bits).min).to(torch.uint8)
        self.qweight = pack_codes(codes, self.w_bits).cpu()

    @torch.inference_mode()
    def unpack(self):
        """Dense (out, in) fp16 weight: normal columns (q + 0.5) * scale, cherry columns copied.
        llama/qlinear.py:120-162."""
        if self.qweight.is_cuda:
            return quant_cuda.unpack_cherryq(self.w_bits, self.qweight, self.cherry_weight, self.cherry_indices,
                                             self.scales, self.in_features, self.group_size)
        codes = unpack_codes(self.qweight, self.w_bits).t()  # (out, Kn)
        q = codes.to(torch.int16 if self.w_bits == 8 else torch.int8) + self.quantizer.iinfo(self.w_bits).min
        s = self.scales.t().repeat_interleave(self.group_size, dim=1)[:, :q.shape[1]]
        normal = self.quantizer.dequantize(q, s)
        weight = torch.zeros(self.out_features, self.in_features, dtype=normal.dtype, device=normal.device)
        weight[..., self._normal_columns(weight.device)] = normal
        weight[..., self.cherry_indices.long()] = self.cherry_weight.t()
        return weight

    # ---- load-time repack (no counterpart in the reference) -----------------------------------
    def _drop_stream(self):
        self._stream = None
        self._released = False

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # new packed buffers: a stream repacked from the old ones is stale
        self._drop_stream()
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() / .cpu(): the stream lives on one device and follows the buffers
        stream = self._stream
        out = super()._apply(fn, *args, **kwargs)
        if stream is not None:
            moved = fn(stream)
            if moved.dtype != torch.uint8 or not moved.is_cuda:
                if self._released:
                    raise RuntimeError("prepack(release_reference=True) left only the weight stream, which exists on "
                                       "its GPU only; call unprepack() before moving or casting the module")
                self._stream = None
            else:
                self._stream = moved
        return out

    def state_dict(self, *args, **kwargs):
        if self._released:
            raise RuntimeError("prepack(release_reference=True) freed the checkpoint-layout buffers; call unprepack() "
                               "before state_dict() / saving")
        return super().state_dict(*args, **kwargs)

    @torch.no_grad()
    def packed_bytes(self) -> int:
        """Bytes of the four checkpoint buffers (codes, scales, cherry rows, cherry indices), also
        while prepack(release_reference=True) holds them only as a weight stream."""
        kn = self.in_features - self.num_cherries
        groups = -(-kn // self.group_size)
        return (kn // 8 * self.w_bits + 2 * groups + 2 * self.num_cherries) * self.out_features + 2 * self.num_cherries

    def prepack(self, release_reference: bool = False):
        """Rearrange the packed buffers, once, into the weight stream the batch-1 kernel of this
        GPU reads fastest (quant_cuda.prepack_cherryq).  The state-dict buffers stay as they are
        unless `release_reference` frees them (unprepack() brings them back, bit for bit).
        Returns True if the layer's shape is taken; otherwise the module is left unchanged and
        keeps using the kernels that read the checkpoint layout."""
        if self.w_bits not in (3, 4) or not self.qweight.is_cuda or self.dequantized:
            return False
        if not quant_cuda.prepack_supported(self.w_bits, 1, self.in_features, self.out_features,
                                            self.num_cherries, self.group_size):
            return False
        self._stream = quant_cuda.prepack_cherryq(self.w_bits, self.qweight, self.cherry_weight, self.cherry_indices,
                                                  self.scales, self.in_features, self.group_size)
        if release_reference:
            dev = self.qweight.device
            self.qweight = torch.empty((0, self.out_features), dtype=torch.uint8, device=dev)
            self.scales = torch.empty((0, self.out_features), dtype=torch.float16, device=dev)
            self.cherry_weight = torch.empty((0, self.out_features), dtype=torch.float16, device=dev)
            self._released = True
        return True

    @torch.no_grad()  # (not inference_mode: the rebuilt buffers must stay loadable with load_state_dict)
    def unprepack(self):
        """Drop the weight stream; if prepack() released the checkpoint-layout buffers, rebuild
        them from it first."""
        stream = self._stream
        if stream is None:
            return
        if self._released:
            (self.cherry_indices, self.cherry_weight, self.qweight,
             self.scales) = quant_cuda.unprepack_cherryq(self.w_bits, stream, self.in_features, self.out_features,
                                                         self.num_cherries, self.group_size)
            self._released = False
        self._stream = None

    # ---- forward ------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, x: torch.Tensor):
        if self._layerwise_dequantize:
            if self.w_bits not in (3, 4):
                raise NotImplementedError(f"{self.w_bits} bit kernel is not implemented yet.")
            if self.dequantized:
                raise RuntimeError("this module was dequantised under dmode(False); its packed buffers are gone")
            out_shape = x.shape[:-1] + (self.out_features,)
            x2 = x.reshape(-1, x.shape[-1])
            if x2.dtype != torch.float16:
                x2 = x2.to(torch.float16)
            x2 = x2.contiguous()
            stream = self._stream
            rows = x2.shape[0]
            # over the repacked stream: one row, and the small batches that measured faster there than on
            # the checkpoint layout's kernels (the matrix-core tile of the one-row kernel filled with real
            # rows: quant_cuda.prepacked_rows_recommended); with the checkpoint buffers released,
            # everything the stream kernels take
            shape = (self.w_bits, rows, self.in_features, self.out_features, self.num_cherries, self.group_size)
            if stream is not None and (rows == 1 or (2 <= rows <= 16 and (
                    quant_cuda.prepack_supported(*shape) if self._released else
                    quant_cuda.prepacked_rows_recommended(*shape)))):
                out = torch.empty(rows, self.out_features, dtype=torch.float16, device=stream.device)
                quant_cuda.matvec_prepacked_cherryq(self.w_bits, x2, stream, out, self.in_features, self.num_cherries)
            elif self._released:
                # only the stream is left: any other number of rows goes over it in pieces of up to 16
                if rows and not quant_cuda.prepack_supported(self.w_bits, min(rows, 16), self.in_features, self.out_features,
                                                             self.num_cherries, self.group_size):
                    raise RuntimeError("prepack(release_reference=True) left only the weight stream, whose kernels do "
                                       "not take this batch size for this layer; call unprepack() first")
                out = torch.empty(rows, self.out_features, dtype=torch.float16, device=stream.device)
                for r0 in range(0, rows, 16):
                    quant_cuda.matvec_prepacked_cherryq(self.w_bits, x2[r0:r0 + 16], stream, out[r0:r0 + 16],
                                                        self.in_features, self.num_cherries)
            elif x2.shape[0] >= self.prefill_rows:
                # prompt-sized batches: one bit-exact dequantisation pass on the GPU into a transient
                # dense weight, then a library fp16 GEMM -- the arithmetic of the dequantised branch
                # below (llama/qlinear.py:183-195) without keeping the dense weight
                out = torch.matmul(x2, self.unpack().t())
            else:
                out = torch.empty(x2.shape[0], self.out_features, dtype=torch.float16, device=self.qweight.device)
                # overwrite mode: no zero-fill launch in front of the kernel (llama/qlinear.py:177)
                quant_cuda.matmul_cherryq(self.w_bits, x2, self.qweight, self.cherry_weight, self.cherry_indices,
                                          self.scales, out, self.group_size, accumulate=False)
            out = out.reshape(out_shape).to(x.dtype)
        else:
            if not self.dequantized:
                self.qweight = self.unpack()
                del self.cherry_indices
                del self.cherry_weight
                del self.scales
                if torch.cuda.is_available():
                    torch.cuda.empty_cache()
                self.dequantized = True
            out = nn.functional.linear(x, self.qweight)
        if self.bias is not None:
            out += self.bias
        return out
