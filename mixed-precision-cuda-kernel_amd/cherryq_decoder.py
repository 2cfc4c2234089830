"""A minimal LLaMA-shaped decoder whose seven per-layer projections are packed CherryQ linears,
for batch-1 greedy decoding on one MI355X.

It reproduces the mathematics of the reference's model (llama/modeling_llama_quant.py: embedding
:949, RMSNorm :75-89, rotary embedding :95-210, attention with KV cache :630-710, gated MLP
:221-251, decoder layer :754-775, final norm + unquantised fp16 lm_head :1064,1132,1222) without
its HF-transformers scaffolding, and the per-token timing loop of benchmark_perplexity.py:92-113.

Every projection is a `llama.qlinear.QuantLinear` (the reference's buffer schema); a token step
calls the fused kernels through `quant_cuda`, and the operations between them (residual +
RMSNorm, rotary + cache write, single-query attention, SiLU * up) through the decode entry points
of libcherryq.  The whole step is captured once in a HIP graph and replayed per token.  q/k/v and
gate/up do not depend on each other: by default each set runs as ONE grouped launch
(`matvec_group`) that also applies the RMSNorm in front of it, rotary + cache write + attention
are one launch, the residual additions are the accumulate mode of o_proj / down_proj, and
SiLU * up is formed inside down_proj: 5 launches per layer.  `grouped=False` keeps one launch per operation;
`fork=True` captures the independent projections of that variant on forked streams, which on this
ROCm stack costs more in cross-stream edges than the overlap gains.
"""
from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch
import torch.nn as nn

import quant_cuda
from llama.qlinear import QuantLinear
from llama.quantizer import FullSymQuantizer

_lib = quant_cuda._lib
_vp, _int, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_lib.cherryq_decode_add_rmsnorm_f16.argtypes = [_vp, _vp, _vp, _vp, _int, _f, _vp]
_lib.cherryq_decode_rope_cache_f16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _f, _vp]
_lib.cherryq_decode_attention_f16.argtypes = [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]
_lib.cherryq_decode_silu_mul_f16.argtypes = [_vp, _vp, _vp, _int, _vp]
_lib.cherryq_decode_argmax_embed_f16.argtypes = [_vp, _int, _vp, _int, _vp, _vp, _vp, _int, _vp, _vp]
_lib.cherryq_decode_argmax_embed_f16.restype = _int
_lib.cherryq_decode_rope_attention_f16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _f, _vp]
_lib.cherryq_decode_attention_max_slices.argtypes = []
_lib.cherryq_decode_attention_max_slices.restype = _int
_lib.cherryq_decode_attention_projection_slices.argtypes = []
_lib.cherryq_decode_attention_projection_slices.restype = _int
_lib.cherryq_decode_rope_attention_split_f16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _int, _int,
                                                         _int, _f, _vp]
_lib.cherryq_decode_rope_attention_split_f16.restype = _int
_lib.cherryq_decode_attention_combine_f16.argtypes = [_vp, _vp, _int, _vp, _int, _int, _vp]
_lib.cherryq_decode_attention_combine_f16.restype = _int
_lib.cherryq_decode_matvec_attention_prepacked_supported.argtypes = [_int, _int, _int, _int]
_lib.cherryq_decode_matvec_attention_prepacked_supported.restype = _int
_lib.cherryq_decode_matvec_attention_prepacked_f16.argtypes = [_int, _vp, _vp, _int, _vp, ctypes.c_size_t, _vp, _int, _int,
                                                               _int, _int, _vp]
_lib.cherryq_decode_matvec_attention_prepacked_f16.restype = _int
_lib.cherryq_decode_head_supported.argtypes = [_int, _int]
_lib.cherryq_decode_head_supported.restype = _int
_lib.cherryq_decode_head_f16.argtypes = [_vp, _vp, _f, _vp, _vp, _int, _int, _vp]
_lib.cherryq_decode_head_f16.restype = _int
for _n in ("cherryq_decode_add_rmsnorm_f16", "cherryq_decode_rope_cache_f16", "cherryq_decode_attention_f16",
           "cherryq_decode_silu_mul_f16", "cherryq_decode_rope_attention_f16"):
    getattr(_lib, _n).restype = _int


class _Layer(ctypes.Structure):
    """struct cherryq_layer of include/cherryq.h"""
    _fields_ = [("qweight", _vp), ("cherry_weight", _vp), ("cherry_indices", _vp), ("scales", _vp), ("mul", _vp),
                ("out_features", _int)]


_lib.cherryq_group_workspace_bytes.argtypes = [_int, ctypes.POINTER(_int)]
_lib.cherryq_group_workspace_bytes.restype = ctypes.c_size_t
_lib.cherryq_decode_matvec_group_f16.argtypes = [_int, _vp, _vp, _vp, _f, ctypes.POINTER(_Layer), _int, _int, _int,
                                                 _int, _int, _vp, ctypes.c_size_t, _vp]
_lib.cherryq_decode_matvec_group_f16.restype = _int


def matvec_group(mods, vec, outs, vec_gate=None, accumulate=False, norm_weight=None, eps=1e-6):
    """outs[i] (+)= act @ W_i^T for 1..4 QuantLinear modules that read the same (1, K) activation
    row, in ONE launch; act = vec, or fp16(fp16(silu(vec_gate)) * vec) when vec_gate is given, or
    norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps)) when norm_weight is given."""
    m0 = mods[0]
    k, c = vec.shape[1], m0.cherry_indices.shape[0]
    for m, o in zip(mods, outs):
        if (m.w_bits, m.group_size, m.cherry_indices.shape[0], m.in_features) != (m0.w_bits, m0.group_size, c, k):
            raise RuntimeError("matvec_group: the layers must share w_bits, group_size, num_cherries and in_features")
        for t, dt in ((m.qweight, torch.uint8), (m.scales, torch.float16), (m.cherry_weight, torch.float16),
                      (m.cherry_indices, torch.int16), (o, torch.float16)):
            if not t.is_cuda or t.dtype != dt or not t.is_contiguous() or t.device != vec.device:
                raise RuntimeError("matvec_group: contiguous GPU tensors of the packed schema's dtypes expected")
        if tuple(o.shape) != (1, m.out_features) or m.qweight.shape != ((k - c) // 8 * m.w_bits, m.out_features):
            raise RuntimeError("matvec_group: buffer shapes do not match the layer")
    if tuple(vec.shape) != (1, k) or vec.dtype != torch.float16 or not vec.is_cuda or not vec.is_contiguous():
        raise RuntimeError("matvec_group: vec must be a contiguous (1, in_features) fp16 GPU tensor")
    if vec_gate is not None and (vec_gate.shape != vec.shape or vec_gate.dtype != torch.float16
                                 or not vec_gate.is_cuda or not vec_gate.is_contiguous()):
        raise RuntimeError("matvec_group: vec_gate must match vec")
    if norm_weight is not None and (tuple(norm_weight.shape) != (k,) or norm_weight.dtype != torch.float16
                                    or not norm_weight.is_cuda or not norm_weight.is_contiguous()):
        raise RuntimeError("matvec_group: norm_weight must be a contiguous (in_features,) fp16 GPU tensor")
    arr = (_Layer * len(mods))(*[_Layer(m.qweight.data_ptr(), quant_cuda._ptr(m.cherry_weight),
                                        quant_cuda._ptr(m.cherry_indices), m.scales.data_ptr(), o.data_ptr(),
                                        m.out_features) for m, o in zip(mods, outs)])
    ns = (_int * len(mods))(*[m.out_features for m in mods])
    stream = _stream()
    ws = quant_cuda._workspace(vec.device, stream, _lib.cherryq_group_workspace_bytes(len(mods), ns))
    _ok(_lib.cherryq_decode_matvec_group_f16(m0.w_bits, vec.data_ptr(), None if vec_gate is None else vec_gate.data_ptr(),
                                             None if norm_weight is None else norm_weight.data_ptr(), eps,
                                             arr, len(mods), k, c, m0.group_size, 1 if accumulate else 0,
                                             ws.data_ptr(), ws.numel(), stream), "matvec_group")


class _StreamLayer(ctypes.Structure):
    _fields_ = [("stream", _vp), ("stream_bytes", ctypes.c_size_t), ("mul", _vp), ("out_features", _int)]


_lib.cherryq_decode_matvec_group_prepacked_f16.argtypes = [_int, _vp, _vp, _f, ctypes.POINTER(_StreamLayer), _int, _int,
                                                           _int, _int, _vp]
_lib.cherryq_decode_matvec_group_prepacked_f16.restype = _int


def matvec_group_prepacked(mods, vec, outs, accumulate=False, norm_weight=None, eps=1e-6):
    """matvec_group for 1..3 QuantLinear modules that hold a repacked weight stream
    (QuantLinear.prepack()): outs[i] (+)= act @ W_i^T in ONE launch without workspace, act = vec or
    norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps))."""
    m0 = mods[0]
    k, c = vec.shape[1], m0.cherry_indices.shape[0]
    for m, o in zip(mods, outs):
        st = getattr(m, "_stream", None)
        if st is None:
            raise RuntimeError("matvec_group_prepacked: every layer must have been prepack()ed")
        if (m.w_bits, m.cherry_indices.shape[0], m.in_features) != (m0.w_bits, c, k):
            raise RuntimeError("matvec_group_prepacked: the layers must share w_bits, num_cherries and in_features")
        if (not o.is_cuda or o.dtype != torch.float16 or not o.is_contiguous() or o.device != vec.device
                or tuple(o.shape) != (1, m.out_features) or st.device != vec.device):
            raise RuntimeError("matvec_group_prepacked: outputs must be contiguous (1, out_features) fp16 tensors on vec's GPU")
    if tuple(vec.shape) != (1, k) or vec.dtype != torch.float16 or not vec.is_cuda or not vec.is_contiguous():
        raise RuntimeError("matvec_group_prepacked: vec must be a contiguous (1, in_features) fp16 GPU tensor")
    if norm_weight is not None and (tuple(norm_weight.shape) != (k,) or norm_weight.dtype != torch.float16
                                    or not norm_weight.is_cuda or not norm_weight.is_contiguous()):
        raise RuntimeError("matvec_group_prepacked: norm_weight must be a contiguous (in_features,) fp16 GPU tensor")
    arr = (_StreamLayer * len(mods))(*[_StreamLayer(m._stream.data_ptr(), m._stream.numel(), o.data_ptr(), m.out_features)
                                       for m, o in zip(mods, outs)])
    _ok(_lib.cherryq_decode_matvec_group_prepacked_f16(m0.w_bits, vec.data_ptr(),
                                                       None if norm_weight is None else norm_weight.data_ptr(), eps, arr,
                                                       len(mods), k, c, 1 if accumulate else 0, _stream()),
        "matvec_group_prepacked")


_lib.cherryq_decode_matvec_gated_prepacked_f16.argtypes = [_int, _vp, _vp, _vp, ctypes.c_size_t, _vp, _int, _int, _int, _int, _vp]
_lib.cherryq_decode_matvec_gated_prepacked_f16.restype = _int


_lib.cherryq_decode_gate_up_prepacked_f16.argtypes = [_int, _vp, _vp, _f, _vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _vp,
                                                      _int, _int, _int, _vp]
_lib.cherryq_decode_gate_up_prepacked_f16.restype = _int
_lib.cherryq_decode_gate_up_prepacked_supported.argtypes = [_int] * 4
_lib.cherryq_decode_gate_up_prepacked_supported.restype = _int


def gate_up_prepacked_supported(gate_mod, up_mod) -> bool:
    """Whether gate_up_prepacked takes this pair of layers (both repacked, same shape and cherry count)."""
    g, u = gate_mod, up_mod
    if getattr(g, "_stream", None) is None or getattr(u, "_stream", None) is None:
        return False
    if (g.w_bits, g.in_features, g.out_features, g.num_cherries) != (u.w_bits, u.in_features, u.out_features, u.num_cherries):
        return False
    return bool(_lib.cherryq_decode_gate_up_prepacked_supported(g.w_bits, g.in_features, g.out_features, g.num_cherries))


def gate_up_prepacked(gate_mod, up_mod, vec, act, norm_weight=None, eps=1e-6):
    """act = fp16(fp16(silu(vec' Wg^T)) * (vec' Wu^T)) in ONE launch over the two repacked layers, vec' =
    vec or norm_weight * fp16(vec * rsqrt(mean(vec^2) + eps)): what the down projection reads."""
    if not gate_up_prepacked_supported(gate_mod, up_mod):
        raise RuntimeError("gate_up_prepacked: two prepack()ed layers of the same supported shape are needed")
    g, u = gate_mod, up_mod
    k, n = g.in_features, g.out_features
    dev = g._stream.device
    for t, shape in ((vec, (1, k)), (act, (1, n))):
        if tuple(t.shape) != shape or t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous() or t.device != dev:
            raise RuntimeError("gate_up_prepacked: vec (1, in_features) and act (1, out_features) must be contiguous fp16 "
                               "tensors on the layers' GPU")
    if norm_weight is not None and (tuple(norm_weight.shape) != (k,) or norm_weight.dtype != torch.float16
                                    or not norm_weight.is_cuda or not norm_weight.is_contiguous()):
        raise RuntimeError("gate_up_prepacked: norm_weight must be a contiguous (in_features,) fp16 GPU tensor")
    _ok(_lib.cherryq_decode_gate_up_prepacked_f16(g.w_bits, vec.data_ptr(), None if norm_weight is None else norm_weight.data_ptr(),
                                                  eps, g._stream.data_ptr(), g._stream.numel(), u._stream.data_ptr(),
                                                  u._stream.numel(), act.data_ptr(), k, n, g.num_cherries, _stream()),
        "gate_up_prepacked")


def matvec_gated_prepacked(mod, vec, vec_gate, out, accumulate=False):
    """out (+)= fp16(fp16(silu(vec_gate)) * vec) @ W^T for a QuantLinear that holds a repacked weight
    stream: the down projection of the gated MLP in one launch, the activation formed while the
    row is staged."""
    st = getattr(mod, "_stream", None)
    if st is None:
        raise RuntimeError("matvec_gated_prepacked: the layer must have been prepack()ed")
    k = mod.in_features
    for t, shape in ((vec, (1, k)), (vec_gate, (1, k)), (out, (1, mod.out_features))):
        if tuple(t.shape) != shape or t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous() or t.device != st.device:
            raise RuntimeError("matvec_gated_prepacked: vec / vec_gate (1, in_features) and out (1, out_features) must be "
                               "contiguous fp16 tensors on the layer's GPU")
    _ok(_lib.cherryq_decode_matvec_gated_prepacked_f16(mod.w_bits, vec.data_ptr(), vec_gate.data_ptr(), st.data_ptr(),
                                                       st.numel(), out.data_ptr(), k, mod.out_features, mod.num_cherries,
                                                       1 if accumulate else 0, _stream()), "matvec_gated_prepacked")


ATTN_SLICES = _lib.cherryq_decode_attention_projection_slices()   # what a repacked output projection combines


def rope_attention_split(q, k, v, k_cache, v_cache, partial, max_sum, pos, n_heads, n_kv_heads, head_dim, max_len,
                         theta, slices=ATTN_SLICES):
    """Rotary embedding + cache write + attention for one token with every head's positions dealt
    to `slices` workgroups: partial (slices, n_heads * head_dim) fp16 and max_sum (slices, n_heads, 2)
    fp32 receive the slices' results (attention_combine / matvec_attention_prepacked read them)."""
    for t, shape, dt in ((q, (1, n_heads * head_dim), torch.float16), (k, (1, n_kv_heads * head_dim), torch.float16),
                         (v, (1, n_kv_heads * head_dim), torch.float16),
                         (k_cache, (n_kv_heads, max_len, head_dim), torch.float16),
                         (v_cache, (n_kv_heads, max_len, head_dim), torch.float16),
                         (partial, (slices, n_heads * head_dim), torch.float16), (max_sum, (slices, n_heads, 2), torch.float32),
                         (pos, (1,), torch.int32)):
        if tuple(t.shape) != shape or t.dtype != dt or not t.is_cuda or not t.is_contiguous() or t.device != q.device:
            raise RuntimeError("rope_attention_split: expected a contiguous %s tensor of shape %s on the GPU, got %s %s"
                               % (dt, shape, t.dtype, tuple(t.shape)))
    _ok(_lib.cherryq_decode_rope_attention_split_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), k_cache.data_ptr(),
                                                     v_cache.data_ptr(), partial.data_ptr(), max_sum.data_ptr(), slices,
                                                     pos.data_ptr(), n_heads, n_kv_heads, head_dim, max_len, theta,
                                                     _stream()), "rope_attention_split")


def attention_combine(partial, max_sum, out, head_dim=128):
    """out (1, n_heads * head_dim) <- the heads' results from the slices' partial results."""
    slices, n = partial.shape
    n_heads = n // head_dim
    for t, shape, dt in ((partial, (slices, n), torch.float16), (max_sum, (slices, n_heads, 2), torch.float32),
                         (out, (1, n), torch.float16)):
        if tuple(t.shape) != shape or t.dtype != dt or not t.is_cuda or not t.is_contiguous() or t.device != partial.device:
            raise RuntimeError("attention_combine: expected a contiguous %s tensor of shape %s on the GPU" % (dt, shape))
    _ok(_lib.cherryq_decode_attention_combine_f16(partial.data_ptr(), max_sum.data_ptr(), slices, out.data_ptr(), n_heads,
                                                  head_dim, _stream()), "attention_combine")


def matvec_attention_prepacked_supported(mod) -> bool:
    return (getattr(mod, "_stream", None) is not None and
            bool(_lib.cherryq_decode_matvec_attention_prepacked_supported(mod.w_bits, mod.in_features, mod.out_features,
                                                                          mod.num_cherries)))


def matvec_attention_prepacked(mod, partial, max_sum, out, accumulate=False):
    """out (+)= heads @ W^T for a QuantLinear that holds a repacked weight stream (the output
    projection), `heads` formed from rope_attention_split's partial results while the row is staged."""
    st = getattr(mod, "_stream", None)
    if st is None:
        raise RuntimeError("matvec_attention_prepacked: the layer must have been prepack()ed")
    k = mod.in_features
    for t, shape, dt in ((partial, (ATTN_SLICES, k), torch.float16), (max_sum, (ATTN_SLICES, k // 128, 2), torch.float32),
                         (out, (1, mod.out_features), torch.float16)):
        if tuple(t.shape) != shape or t.dtype != dt or not t.is_cuda or not t.is_contiguous() or t.device != st.device:
            raise RuntimeError("matvec_attention_prepacked: expected a contiguous %s tensor of shape %s on the layer's GPU"
                               % (dt, shape))
    _ok(_lib.cherryq_decode_matvec_attention_prepacked_f16(mod.w_bits, partial.data_ptr(), max_sum.data_ptr(), ATTN_SLICES,
                                                           st.data_ptr(), st.numel(), out.data_ptr(), k, mod.out_features,
                                                           mod.num_cherries, 1 if accumulate else 0, _stream()),
        "matvec_attention_prepacked")


def _group(mods, vec, outs, accumulate=False, norm_weight=None, eps=1e-6):
    """The grouped launch over whichever layout the layers hold: the repacked streams when every
    layer of the group has one, the checkpoint layout otherwise."""
    if all(getattr(m, "_stream", None) is not None for m in mods):
        matvec_group_prepacked(mods, vec, outs, accumulate=accumulate, norm_weight=norm_weight, eps=eps)
    else:
        matvec_group(mods, vec, outs, accumulate=accumulate, norm_weight=norm_weight, eps=eps)


def _ok(rc, what):
    if rc != 0:
        quant_cuda._fail(rc, what)


def _stream():
    return quant_cuda._current_stream(torch.cuda.current_device())


@dataclass
class DecoderConfig:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 256
    w_bits: int = 4
    group_size: int = 128
    cherry_fraction: float = 1 / 256

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads


def random_packed_linear(cfg: DecoderConfig, in_features, out_features, gen: torch.Generator, device) -> QuantLinear:
    """A QuantLinear with random but well-formed packed buffers, generated on the device:
    uniform codes, scales such that the dequantised weights have a standard deviation of about
    0.02 (LLaMA's init), sorted random cherry columns with N(0, 0.02) fp16 weights."""
    q = QuantLinear(cfg.w_bits, cfg.group_size, FullSymQuantizer, cfg.cherry_fraction, in_features, out_features,
                    bias=False)
    c = q.num_cherries
    code_std = math.sqrt((4 ** cfg.w_bits - 1) / 12.0)
    q.qweight = torch.randint(0, 256, q.qweight.shape, dtype=torch.uint8, device=device, generator=gen)
    q.scales = ((torch.rand(q.scales.shape, device=device, generator=gen) * 0.5 + 0.75) * (0.02 / code_std)).half()
    q.cherry_weight = (torch.randn(q.cherry_weight.shape, device=device, generator=gen) * 0.02).half()
    q.cherry_indices = torch.randperm(in_features, device=device, generator=gen)[:c].sort().values.to(torch.int16)
    return q


class DecoderLayer(nn.Module):
    def __init__(self, cfg: DecoderConfig, gen, device):
        super().__init__()
        h, kv = cfg.hidden_size, cfg.num_key_value_heads * cfg.head_dim
        self.q_proj = random_packed_linear(cfg, h, h, gen, device)
        self.k_proj = random_packed_linear(cfg, h, kv, gen, device)
        self.v_proj = random_packed_linear(cfg, h, kv, gen, device)
        self.o_proj = random_packed_linear(cfg, h, h, gen, device)
        self.gate_proj = random_packed_linear(cfg, h, cfg.intermediate_size, gen, device)
        self.up_proj = random_packed_linear(cfg, h, cfg.intermediate_size, gen, device)
        self.down_proj = random_packed_linear(cfg, cfg.intermediate_size, h, gen, device)
        self.input_layernorm = nn.Parameter(torch.ones(h, dtype=torch.float16, device=device), requires_grad=False)
        self.post_attention_layernorm = nn.Parameter(torch.ones(h, dtype=torch.float16, device=device),
                                                     requires_grad=False)


class CherryLlamaDecoder(nn.Module):
    """Random-init decoder; `generate()` does greedy decoding with a captured token step."""

    def __init__(self, cfg: DecoderConfig, seed: int = 0, device="cuda"):
        super().__init__()
        self.cfg = cfg
        self.device_ = torch.device(device)
        if cfg.head_dim * cfg.num_attention_heads != cfg.hidden_size:
            raise ValueError("hidden_size must be num_attention_heads * head_dim")
        if not _lib.cherryq_decode_head_supported(cfg.vocab_size, cfg.hidden_size):
            raise ValueError("hidden_size must be a multiple of 8, at most 8192 (the head kernel's range)")
        gen = torch.Generator(device=self.device_).manual_seed(seed)
        h = cfg.hidden_size
        self.embed_tokens = (torch.randn(cfg.vocab_size, h, device=self.device_, generator=gen) * 0.02).half()
        self.layers = nn.ModuleList([DecoderLayer(cfg, gen, self.device_) for _ in range(cfg.num_hidden_layers)])
        self.norm = torch.ones(h, dtype=torch.float16, device=self.device_)
        self.lm_head = (torch.randn(cfg.vocab_size, h, device=self.device_, generator=gen) * 0.02).half()
        L, kvh, ml, hd = cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.max_position_embeddings, cfg.head_dim
        self.k_cache = torch.zeros(L, kvh, ml, hd, dtype=torch.float16, device=self.device_)
        self.v_cache = torch.zeros_like(self.k_cache)
        # static step buffers (a captured graph replays on fixed addresses)
        f16 = dict(dtype=torch.float16, device=self.device_)
        self.pos = torch.zeros(1, dtype=torch.int32, device=self.device_)
        self.token = torch.zeros(1, dtype=torch.int64, device=self.device_)
        self.next_token = torch.zeros(1, dtype=torch.int64, device=self.device_)
        self.hid = torch.zeros(1, h, **f16)
        self.normed = torch.zeros(1, h, **f16)
        self.q = torch.zeros(1, h, **f16)
        self.k = torch.zeros(1, kvh * hd, **f16)
        self.v = torch.zeros(1, kvh * hd, **f16)
        self.attn = torch.zeros(1, h, **f16)
        self.proj = torch.zeros(1, h, **f16)
        self.gate = torch.zeros(1, cfg.intermediate_size, **f16)
        self.up = torch.zeros(1, cfg.intermediate_size, **f16)
        self.act = torch.zeros(1, cfg.intermediate_size, **f16)
        self.attn_part = torch.zeros(ATTN_SLICES, h, **f16)   # split attention: the slices' results ...
        self.attn_ml = torch.zeros(ATTN_SLICES, cfg.num_attention_heads, 2, dtype=torch.float32, device=self.device_)  # ... and (maximum, sum)
        self.logits16 = torch.zeros(1, cfg.vocab_size, **f16)
        self.history = torch.zeros(ml, dtype=torch.int64, device=self.device_)  # history[p]: token predicted at position p
        self._graph = None
        self.fuse_norm = True
        self.fuse_head = True  # final RMSNorm inside the head launch (False: a launch of its own in front)
        # Attention dealt to ATTN_SLICES workgroups per head, combined by a repacked o_proj's staging: None =
        # for caches of 1024 positions and more.  (Measured per layer: 256-position cache 5.5 -> 5.0 us for
        # the attention but 4.3 -> 6.5 us for the projection; 1000 of 4096 positions 18.1 -> 11.3 us, 4000
        # positions 50 -> 22 us for the attention.)
        self.split_attn = None
        self.fuse_act = True   # gate / up as one launch that stores SiLU(gate) * up (layers repacked), plain down projection
        self.layer_trace = None
        self._side = [torch.cuda.Stream(device=self.device_) for _ in range(2)] if self.device_.type == "cuda" else []

    # ---- checkpoint schema of the reference's LlamaForCausalLM (llama/modeling_llama_quant.py:
    # model.embed_tokens :949, layers.N.self_attn.{q,k,v,o}_proj :299-310, layers.N.mlp.{gate,up,
    # down}_proj :221-229, the two layer norms :754-775, model.norm :1064, lm_head :1132), with the
    # packed buffer names of llama/qlinear.py:43-63, as utils.py:99-118 writes it
    _ATTN = ("q_proj", "k_proj", "v_proj", "o_proj")
    _MLP = ("gate_proj", "up_proj", "down_proj")
    _BUFFERS = ("cherry_indices", "cherry_weight", "qweight", "scales")

    def reference_state_dict(self) -> dict:
        sd = {"model.embed_tokens.weight": self.embed_tokens}
        for i, layer in enumerate(self.layers):
            for group, names in (("self_attn", self._ATTN), ("mlp", self._MLP)):
                for n in names:
                    m = getattr(layer, n)
                    for b in self._BUFFERS:
                        sd[f"model.layers.{i}.{group}.{n}.{b}"] = getattr(m, b)
            sd[f"model.layers.{i}.input_layernorm.weight"] = layer.input_layernorm.data
            sd[f"model.layers.{i}.post_attention_layernorm.weight"] = layer.post_attention_layernorm.data
        sd["model.norm.weight"] = self.norm
        sd["lm_head.weight"] = self.lm_head
        return sd

    def load_reference_state_dict(self, sd: dict):
        """Copy a checkpoint in the reference's schema into this decoder (shapes and dtypes are
        checked; rotary inv_freq buffers, which older transformers versions persist, are ignored)."""
        want = self.reference_state_dict()
        extra = [k for k in sd if k not in want and not k.endswith("rotary_emb.inv_freq")]
        missing = [k for k in want if k not in sd]
        if extra or missing:
            raise KeyError(f"checkpoint does not match the decoder: missing {missing[:4]}, unexpected {extra[:4]}")
        for k, dst in want.items():
            src = sd[k]
            if tuple(src.shape) != tuple(dst.shape) or src.dtype != dst.dtype:
                raise ValueError(f"{k}: checkpoint has {tuple(src.shape)} {src.dtype}, "
                                 f"decoder expects {tuple(dst.shape)} {dst.dtype}")
            dst.copy_(src)
        for layer in self.layers:  # streams repacked from the previous weights are stale
            for m in layer.children():
                m._stream = None
        self._graph = None

    def prepack(self, only_recommended=True, release_reference=False):
        """Repack, once, every linear whose shape the library recommends it for (on MI355X: all
        seven projections of the LLaMA-7B, -13B and -70B shapes) into the weight stream the batch-1
        kernel reads fastest; the token step then uses the stream kernels for them.  The
        checkpoint-layout buffers stay (the batched prompt pass reads them) unless
        `release_reference` frees them: one copy of the weights in memory, the prompt pass then goes
        over the streams 16 rows at a time, and state_dict() needs unprepack() first.  Returns the
        number of layers repacked."""
        n = 0
        for layer in self.layers:
            for m in layer.children():
                if only_recommended and not quant_cuda.prepack_recommended(m.w_bits, m.in_features, m.out_features,
                                                                           m.num_cherries, m.group_size):
                    continue
                n += bool(m.prepack(release_reference=release_reference))
        self._graph = None
        return n

    def unprepack(self):
        for layer in self.layers:
            for m in layer.children():
                m.unprepack()
        self._graph = None

    # ---- packed bytes a token step must read (for the roofline of tokens/s)
    def step_bytes(self) -> int:
        n = self.lm_head.numel() * 2
        for layer in self.layers:
            for m in layer.children():
                n += m.packed_bytes()
        return n

    def _linear(self, m: QuantLinear, x, out):
        if getattr(m, "_released", False):  # only the weight stream is left
            quant_cuda.matvec_prepacked_cherryq(m.w_bits, x, m._stream, out, m.in_features, m.num_cherries)
            return
        quant_cuda.matmul_cherryq(m.w_bits, x, m.qweight, m.cherry_weight, m.cherry_indices, m.scales, out,
                                  m.group_size, accumulate=False)

    def _fork(self, fns):
        """Run independent launches on forked streams (inside a capture this becomes a fork/join)."""
        main = torch.cuda.current_stream()
        fns[0]()
        for fn, st in zip(fns[1:], self._side):
            st.wait_stream(main)
            with torch.cuda.stream(st):
                fn()
        for st in self._side[:len(fns) - 1]:
            main.wait_stream(st)

    def _norm(self, weight, delta=None):
        cfg = self.cfg
        _ok(_lib.cherryq_decode_add_rmsnorm_f16(self.hid.data_ptr(), delta, weight.data_ptr(), self.normed.data_ptr(),
                                                cfg.hidden_size, cfg.rms_norm_eps, _stream()), "add_rmsnorm")

    def _step_grouped(self):
        """The token step with 5 launches per layer: RMSNorm + q/k/v in one grid, rotary + cache
        write + attention in one, o_proj accumulating into the hidden state (the residual add,
        rounded once from fp32), RMSNorm + gate/up in one grid, down_proj with SiLU * up formed in
        its activation staging and accumulating into the hidden state.  `self.fuse_norm = False`
        keeps the two norms as launches of their own (7 per layer)."""
        cfg = self.cfg
        nh, nkv, hd, ml = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.max_position_embeddings
        for li, layer in enumerate(self.layers):
            qkv, gu = [layer.q_proj, layer.k_proj, layer.v_proj], [layer.gate_proj, layer.up_proj]
            if self.fuse_norm:
                _group(qkv, self.hid, [self.q, self.k, self.v], norm_weight=layer.input_layernorm,
                       eps=cfg.rms_norm_eps)
            else:
                self._norm(layer.input_layernorm)
                _group(qkv, self.normed, [self.q, self.k, self.v])
            split = ml >= 1024 if self.split_attn is None else self.split_attn
            if split and hd == 128 and matvec_attention_prepacked_supported(layer.o_proj):
                # every head's positions on ATTN_SLICES compute units; o_proj combines the slices' results
                # while it stages its row
                rope_attention_split(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], self.attn_part,
                                     self.attn_ml, self.pos, nh, nkv, hd, ml, cfg.rope_theta)
                matvec_attention_prepacked(layer.o_proj, self.attn_part, self.attn_ml, self.hid, accumulate=True)
            else:
                _ok(_lib.cherryq_decode_rope_attention_f16(self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(),
                                                           self.k_cache[li].data_ptr(), self.v_cache[li].data_ptr(),
                                                           self.attn.data_ptr(), self.pos.data_ptr(), nh, nkv, hd, ml,
                                                           cfg.rope_theta, _stream()), "rope_attention")
                _group([layer.o_proj], self.attn, [self.hid], accumulate=True)
            down = layer.down_proj
            if self.fuse_act and getattr(down, "_stream", None) is not None and gate_up_prepacked_supported(*gu):
                # gate / up in one launch that stores SiLU(gate) * up, then the plain down projection
                if self.fuse_norm:
                    gate_up_prepacked(gu[0], gu[1], self.hid, self.act, norm_weight=layer.post_attention_layernorm,
                                      eps=cfg.rms_norm_eps)
                else:
                    self._norm(layer.post_attention_layernorm)
                    gate_up_prepacked(gu[0], gu[1], self.normed, self.act)
                matvec_group_prepacked([down], self.act, [self.hid], accumulate=True)
            else:
                if self.fuse_norm:
                    _group(gu, self.hid, [self.gate, self.up], norm_weight=layer.post_attention_layernorm,
                           eps=cfg.rms_norm_eps)
                else:
                    self._norm(layer.post_attention_layernorm)
                    _group(gu, self.normed, [self.gate, self.up])
                # the down projection forms SiLU(gate) * up while it stages its row: split-K workgroups of the
                # checkpoint layout each do so for their own slice only (over a weight stream every workgroup
                # would repeat it for the whole row: measured 9.9 us against 8.0)
                matvec_group([down], self.up, [self.hid], vec_gate=self.gate, accumulate=True)
            if self.layer_trace is not None:  # validation only (eager runs): the hidden state after every layer
                self.layer_trace.append(self.hid.clone())
        if self.fuse_head:
            self._head(self.hid, self.norm)
        else:
            self._norm(self.norm)
            self._head(self.normed, None)

    def _head(self, row, norm_weight):
        """Unquantised fp16 head over `row` (the final RMSNorm applied inside the launch when
        norm_weight is given), then the greedy tail on the device: next_token = argmax, recorded
        in history[pos]; its embedding becomes the next step's hidden state; pos += 1."""
        cfg = self.cfg
        _ok(_lib.cherryq_decode_head_f16(row.data_ptr(), norm_weight.data_ptr() if norm_weight is not None else None,
                                         cfg.rms_norm_eps, self.lm_head.data_ptr(), self.logits16.data_ptr(),
                                         cfg.vocab_size, cfg.hidden_size, _stream()), "head")
        _ok(_lib.cherryq_decode_argmax_embed_f16(self.logits16.data_ptr(), cfg.vocab_size, self.embed_tokens.data_ptr(),
                                                 cfg.hidden_size, self.hid.data_ptr(), self.next_token.data_ptr(),
                                                 self.history.data_ptr(), self.history.numel(), self.pos.data_ptr(),
                                                 _stream()), "argmax_embed")

    @property
    def logits(self):
        return self.logits16.float()

    def embed(self):
        """hid <- embedding of self.token.  A step reads its input from `hid`: after a step `hid`
        already holds the embedding of the token that step predicted, so free-running greedy
        decoding needs no call here; feeding a given token (prompt, teacher forcing) does."""
        torch.index_select(self.embed_tokens, 0, self.token, out=self.hid)

    def _step(self, fork=False, grouped=True):
        """One token: the embedding in self.hid at position self.pos -> self.logits16, self.next_token,
        the next input in self.hid; pos += 1.
        grouped=False runs every projection and every element-wise operation as its own launch
        (12 per layer), the literal sequence of the reference's decoder layer."""
        if grouped and not fork:
            return self._step_grouped()
        cfg = self.cfg
        nh, nkv, hd, ml = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.max_position_embeddings
        delta = None
        for li, layer in enumerate(self.layers):
            _ok(_lib.cherryq_decode_add_rmsnorm_f16(self.hid.data_ptr(), delta, layer.input_layernorm.data_ptr(),
                                                    self.normed.data_ptr(), cfg.hidden_size, cfg.rms_norm_eps,
                                                    _stream()), "add_rmsnorm")
            qkv = [lambda l=layer: self._linear(l.q_proj, self.normed, self.q),
                   lambda l=layer: self._linear(l.k_proj, self.normed, self.k),
                   lambda l=layer: self._linear(l.v_proj, self.normed, self.v)]
            if fork:
                self._fork(qkv)
            else:
                for fn in qkv:
                    fn()
            _ok(_lib.cherryq_decode_rope_cache_f16(self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(),
                                                   self.k_cache[li].data_ptr(), self.v_cache[li].data_ptr(),
                                                   self.pos.data_ptr(), nh, nkv, hd, ml, cfg.rope_theta, _stream()),
                "rope_cache")
            _ok(_lib.cherryq_decode_attention_f16(self.q.data_ptr(), self.k_cache[li].data_ptr(),
                                                  self.v_cache[li].data_ptr(), self.attn.data_ptr(),
                                                  self.pos.data_ptr(), nh, nkv, hd, ml, _stream()), "attention")
            self._linear(layer.o_proj, self.attn, self.proj)
            _ok(_lib.cherryq_decode_add_rmsnorm_f16(self.hid.data_ptr(), self.proj.data_ptr(),
                                                    layer.post_attention_layernorm.data_ptr(), self.normed.data_ptr(),
                                                    cfg.hidden_size, cfg.rms_norm_eps, _stream()), "add_rmsnorm")
            gu = [lambda l=layer: self._linear(l.gate_proj, self.normed, self.gate),
                  lambda l=layer: self._linear(l.up_proj, self.normed, self.up)]
            if fork:
                self._fork(gu)
            else:
                for fn in gu:
                    fn()
            _ok(_lib.cherryq_decode_silu_mul_f16(self.gate.data_ptr(), self.up.data_ptr(), self.act.data_ptr(),
                                                 cfg.intermediate_size, _stream()), "silu_mul")
            self._linear(layer.down_proj, self.act, self.proj)
            delta = self.proj.data_ptr()
        _ok(_lib.cherryq_decode_add_rmsnorm_f16(self.hid.data_ptr(), delta, self.norm.data_ptr(),
                                                self.normed.data_ptr(), cfg.hidden_size, cfg.rms_norm_eps, _stream()),
            "final norm")
        self._head(self.normed, None)

    def reset(self):
        self.pos.zero_()
        self.k_cache.zero_()
        self.v_cache.zero_()

    def capture(self, fork=False, grouped=True):
        """Warm up (allocates the per-stream workspaces) and capture one token step."""
        self.reset()
        s = torch.cuda.Stream(device=self.device_)
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                self._step(fork, grouped)
            s.synchronize()
            self._graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self._graph, stream=s):
                self._step(fork, grouped)
        torch.cuda.current_stream().wait_stream(s)
        self.reset()

    @torch.inference_mode()
    def prefill(self, prompt_ids: torch.Tensor) -> torch.Tensor:
        """The whole prompt in one batched pass, as the reference's model processes it
        (llama/modeling_llama_quant.py:1009-1100): every linear sees all T rows at once (the tiled
        GEMM kernel from 17 rows, the small-batch kernel below), RMSNorm / rotary / causal attention
        are torch operations with the reference's rounding points.  Fills the KV caches for
        positions 0..T-1, leaves the decoder exactly where T token steps would (position T, the
        first generated token predicted and embedded) and returns the last position's logits."""
        cfg = self.cfg
        ids = prompt_ids.to(self.device_)
        T, nh, nkv, hd = ids.numel(), cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        assert ids.dim() == 1 and 1 <= T <= cfg.max_position_embeddings

        def norm(x, w):
            xf = x.float()
            return w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps)).half()

        pos = torch.arange(T, device=self.device_, dtype=torch.float32)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2, device=self.device_, dtype=torch.float32) / hd))
        fr = torch.outer(pos, inv)
        emb = torch.cat([fr, fr], dim=-1)
        cos, sin = emb.cos().half()[None], emb.sin().half()[None]  # (1, T, hd)

        def rot(x):
            return torch.cat([-x[..., hd // 2:], x[..., :hd // 2]], dim=-1)

        self.reset()
        h = self.embed_tokens[ids]
        mask = torch.full((T, T), float("-inf"), device=self.device_).triu(1)
        rep = nh // nkv
        for li, layer in enumerate(self.layers):
            x = norm(h, layer.input_layernorm)
            q = layer.q_proj(x).view(T, nh, hd).transpose(0, 1)
            k = layer.k_proj(x).view(T, nkv, hd).transpose(0, 1)
            v = layer.v_proj(x).view(T, nkv, hd).transpose(0, 1)
            q = q * cos + rot(q) * sin
            k = k * cos + rot(k) * sin
            self.k_cache[li, :, :T].copy_(k)
            self.v_cache[li, :, :T].copy_(v)
            kk, vv = k.repeat_interleave(rep, 0), v.repeat_interleave(rep, 0)
            att = (q @ kk.transpose(1, 2)) / math.sqrt(hd)
            att = torch.softmax(att.float() + mask, dim=-1).half()
            a = (att @ vv).transpose(0, 1).reshape(T, nh * hd)
            h = h + layer.o_proj(a)
            x = norm(h, layer.post_attention_layernorm)
            h = h + layer.down_proj(torch.nn.functional.silu(layer.gate_proj(x)) * layer.up_proj(x))
        self.normed.copy_(norm(h[T - 1:T], self.norm))
        self.pos.fill_(T - 1)
        self._head(self.normed, None)  # logits of the last prompt position; greedy tail: history[T-1], next embedding, pos = T
        return self.logits

    @torch.inference_mode()
    def generate(self, prompt_ids: torch.Tensor, max_new_tokens: int, use_graph=True, sync_each_token=False,
                 batched_prefill=False):
        """Greedy decoding.  The prompt is fed token by token through the same step, or, with
        batched_prefill, in one pass over all prompt rows (prefill is not part of the timed
        region either way).  Returns (generated ids, per-token seconds of the decode part when
        sync_each_token, total decode seconds)."""
        import time
        assert prompt_ids.dim() == 1 and prompt_ids.numel() + max_new_tokens <= self.cfg.max_position_embeddings
        if use_graph and self._graph is None:
            self.capture()
        self.reset()
        run = self._graph.replay if use_graph else self._step
        prompt_ids = prompt_ids.to(self.device_)
        n_prompt = prompt_ids.numel()
        if batched_prefill:
            self.prefill(prompt_ids)
        else:
            for i in range(n_prompt):
                self.token.copy_(prompt_ids[i:i + 1])
                self.embed()
                run()
        torch.cuda.synchronize()
        times = []
        t0 = time.perf_counter()
        for i in range(max_new_tokens):
            tick = time.perf_counter()
            run()  # consumes the token the previous step predicted; nothing for the host to do
            if sync_each_token:
                torch.cuda.synchronize()
                times.append(time.perf_counter() - tick)
        torch.cuda.synchronize()
        total = time.perf_counter() - t0
        # history[p] is the token predicted at position p: the first generated token was predicted
        # by the last prompt step
        out = self.history[n_prompt - 1:n_prompt - 1 + max_new_tokens].clone()
        return out, times, total

    @torch.inference_mode()
    def step_logits(self, ids: torch.Tensor, use_graph=False, fork=False, grouped=True) -> torch.Tensor:
        """Logits after each token of `ids`, produced by the token step (teacher forcing)."""
        if use_graph and self._graph is None:
            self.capture(fork, grouped)
        self.reset()
        ids = ids.to(self.device_)
        rows = []
        for i in range(ids.numel()):
            self.token.copy_(ids[i:i + 1])
            self.embed()
            if use_graph:
                self._graph.replay()
            else:
                self._step(fork, grouped)
            rows.append(self.logits)
        torch.cuda.synchronize()
        return torch.cat(rows, dim=0)

    # ---- reference: same model with dense fp16 weights and plain torch ops -------------------
    @torch.inference_mode()
    def reference_logits(self, ids: torch.Tensor) -> torch.Tensor:
        """Logits for every position of `ids` (teacher forcing) from dequantised weights and torch
        operations only (fp32 softmax/norm as in the reference's eager path)."""
        cfg = self.cfg
        ids = ids.to(self.device_)
        T, nh, nkv, hd = ids.numel(), cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim

        def norm(x, w):
            xf = x.float()
            return w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps)).half()

        pos = torch.arange(T, device=self.device_, dtype=torch.float32)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2, device=self.device_, dtype=torch.float32) / hd))
        fr = torch.outer(pos, inv)
        emb = torch.cat([fr, fr], dim=-1)
        cos, sin = emb.cos().half()[None], emb.sin().half()[None]  # (1, T, hd)

        def rot(x):
            x1, x2 = x[..., :hd // 2], x[..., hd // 2:]
            return torch.cat([-x2, x1], dim=-1)

        h = self.embed_tokens[ids]
        mask = torch.full((T, T), float("-inf"), device=self.device_).triu(1)
        for layer in self.layers:
            dense = {n: m.unpack() for n, m in layer.named_children()}
            x = norm(h, layer.input_layernorm)
            q = (x @ dense["q_proj"].t()).view(T, nh, hd).transpose(0, 1)
            k = (x @ dense["k_proj"].t()).view(T, nkv, hd).transpose(0, 1)
            v = (x @ dense["v_proj"].t()).view(T, nkv, hd).transpose(0, 1)
            q = q * cos + rot(q) * sin
            k = k * cos + rot(k) * sin
            rep = nh // nkv
            k, v = k.repeat_interleave(rep, 0), v.repeat_interleave(rep, 0)
            att = (q @ k.transpose(1, 2)) / math.sqrt(hd)
            att = torch.softmax(att.float() + mask, dim=-1).half()
            a = (att @ v).transpose(0, 1).reshape(T, nh * hd)
            h = h + a @ dense["o_proj"].t()
            x = norm(h, layer.post_attention_layernorm)
            m = torch.nn.functional.silu(x @ dense["gate_proj"].t()) * (x @ dense["up_proj"].t())
            h = h + m @ dense["down_proj"].t()
        return (norm(h, self.norm) @ self.lm_head.t()).float()
