"""CPU oracle for CherryQ's mixed-precision quantized linear (numpy).

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU, the algorithm of the
reference operator so that the HIP path can be checked against it.  It must never be
imported by the product package; only tests, the smoke check and the `cpu_baseline`
leg of the benchmark may use it.

Every function cites the reference lines it follows (paths relative to the reference
repository root).  Arithmetic that the reference performs on fp16 torch tensors is
restated with explicit float32 intermediates and a single rounding to float16, which is
how torch evaluates fp16 element-wise ops on the CPU.

Parity status: every function below is pinned by the golden vectors produced from the
reference's own Python (tests/golden/) and by closed-form / brute-force checks in
tests/test_oracle_*.py, except `fused_reference_order`, which restates the CUDA
kernels' evaluation order and is pinned only against the dense formulation
(the CUDA code cannot run here): parity unpinned against the CUDA binary itself.
"""
from __future__ import annotations

import math

import numpy as np

F16 = np.float16
F32 = np.float32


# --------------------------------------------------------------------------- schema

def iinfo(w_bits: int) -> tuple[int, int]:
    """Integer range of the full symmetric grid.  llama/quantizer.py:141-146."""
    return -(2 ** (w_bits - 1)), 2 ** (w_bits - 1) - 1


def num_cherries(in_features: int, cherry_fraction: float = 1 / 256) -> int:
    """llama/qlinear.py:37, llama/cherry_linear.py:33."""
    return math.ceil(in_features * cherry_fraction) // 8 * 8


def buffer_shapes(w_bits, group_size, in_features, out_features, cherry_fraction=1 / 256):
    """Shapes/dtypes of the packed operand set.  llama/qlinear.py:25-65."""
    g = group_size if group_size != -1 else in_features
    c = num_cherries(in_features, cherry_fraction)
    kn = in_features - c
    return {
        "cherry_indices": ((c,), np.int16),
        "cherry_weight": ((c, out_features), F16),
        "qweight": ((kn // 8 * w_bits, out_features), np.uint8),
        "scales": ((math.ceil(kn / g), out_features), F16),
    }


def normal_indices(in_features: int, cherry_indices) -> np.ndarray:
    """Ascending complement of the cherry columns.  llama/qlinear.py:75-76."""
    mask = np.ones(in_features, dtype=bool)
    mask[np.asarray(cherry_indices, dtype=np.int64)] = False
    return np.nonzero(mask)[0]


def gather_offset(k, cherry_indices) -> np.ndarray:
    """`low(k)` of the CUDA kernels: upper bound of k in (idx[m] - m).

    csrc/quant_cuda_kernel.cu:785-795.  normal_indices[k] == k + low(k).
    """
    idx = np.asarray(cherry_indices, dtype=np.int64)
    t = idx - np.arange(idx.shape[0])
    return np.searchsorted(t, np.asarray(k, dtype=np.int64), side="right")


# --------------------------------------------------------------------------- quantizer

def get_scaling_factor(w_group: np.ndarray, w_bits: int) -> np.ndarray:
    """Per-row scale of one group: (max|w| + 1e-6) / 2^(b-1), keepdim.

    llama/quantizer.py:148-152 with get_max_input (10-34, row-wise branch).  The
    arithmetic runs in the weight dtype; for fp16 weights torch computes each op in
    float32 and rounds the result to fp16.
    """
    dt = w_group.dtype
    mx = np.max(np.abs(w_group), axis=-1, keepdims=True)
    if dt == F16:
        s = (mx.astype(F32) + F32(1e-6)).astype(F16)
        s = (s.astype(F32) / F32(2 ** (w_bits - 1))).astype(F16)
        return s
    return ((mx + dt.type(1e-6)) / dt.type(2 ** (w_bits - 1))).astype(dt)


def get_scaling_factors(normal_weight: np.ndarray, w_bits: int, group_size: int) -> np.ndarray:
    """(out, num_group) scales over compacted normal columns.  llama/cherry_linear.py:69-75."""
    cols = []
    for i in range(0, normal_weight.shape[-1], group_size):
        cols.append(get_scaling_factor(normal_weight[:, i:i + group_size], w_bits))
    return np.concatenate(cols, axis=-1)


def expand_scales(s: np.ndarray, group_size: int, width: int) -> np.ndarray:
    """repeat_interleave along the last axis, cut to width.  llama/qlinear.py:81."""
    return np.repeat(s, group_size, axis=-1)[..., :width]


def _div_in_dtype(w: np.ndarray, s: np.ndarray) -> np.ndarray:
    if w.dtype == F16:
        with np.errstate(all="ignore"):
            return (w.astype(F32) / s.astype(F32)).astype(F16)
    return w / s


def quantize(w: np.ndarray, s: np.ndarray, w_bits: int) -> np.ndarray:
    """FullSymQuantizer.quantize.  llama/quantizer.py:154-158.

    (w / s) in the weight dtype, then float32: clamp to +-(2^(b-1) - 0.01), minus 0.5,
    round half to even, int32.
    """
    qmax = F32(2 ** (w_bits - 1) - 1e-2)
    r = _div_in_dtype(w, np.broadcast_to(s, w.shape)).astype(F32)
    r = np.clip(r, -qmax, qmax) - F32(0.5)
    return np.rint(r).astype(np.int32)


def dequantize(q: np.ndarray, s: np.ndarray) -> np.ndarray:
    """FullSymQuantizer.dequantize: (q.to(s.dtype) + 0.5) * s.  llama/quantizer.py:160-163."""
    dt = s.dtype
    if dt == F16:
        a = (q.astype(F16).astype(F32) + F32(0.5)).astype(F16)
        with np.errstate(all="ignore"):
            return (a.astype(F32) * np.broadcast_to(s, q.shape).astype(F32)).astype(F16)
    return (q.astype(dt) + dt.type(0.5)) * s


def transform(w: np.ndarray, s: np.ndarray, w_bits: int) -> np.ndarray:
    """FullSymQuantizer.transform (fake quantisation in the weight dtype).

    llama/quantizer.py:165-170.  Every op is evaluated in w.dtype; for fp16 the clamp
    bounds are the fp16 roundings of +-(2^(b-1) - 0.01).
    """
    dt = w.dtype
    s = np.broadcast_to(s, w.shape)
    qmax = 2 ** (w_bits - 1) - 1e-2
    if dt == F16:
        r = _div_in_dtype(w, s)
        r = np.clip(r, F16(-qmax), F16(qmax))
        r = (r.astype(F32) - F32(0.5)).astype(F16)
        r = np.rint(r.astype(F32)).astype(F16)
        r = (r.astype(F32) + F32(0.5)).astype(F16)
        with np.errstate(all="ignore"):
            return (r.astype(F32) * s.astype(F32)).astype(F16)
    r = np.clip(w / s, dt.type(-qmax), dt.type(qmax))
    return (np.rint(r - dt.type(0.5)) + dt.type(0.5)) * s


# --------------------------------------------------------------------------- bit layout

def pack_codes(u: np.ndarray, w_bits: int) -> np.ndarray:
    """Pack codes u (Kn, N) uint8 in [0, 2^b) into qweight (Kn/8*b, N) uint8.

    llama/qlinear.py:86-116.  b in {2,4,8}: row r holds u[(8/b) r + t] << (b t).
    b == 3: each 8 codes of a column form a little-endian 24-bit word
    sum(u[8t+i] << 3i) stored in three consecutive byte rows.
    """
    kn, n = u.shape
    u = u.astype(np.uint32)
    if w_bits in (2, 4, 8):
        per = 8 // w_bits
        assert kn % per == 0
        q = np.zeros((kn // per, n), dtype=np.uint32)
        for t in range(per):
            q |= u[t::per] << (w_bits * t)
        return q.astype(np.uint8)
    if w_bits == 3:
        assert kn % 8 == 0
        units = u.reshape(kn // 8, 8, n)
        w24 = np.zeros((kn // 8, n), dtype=np.uint32)
        for i in range(8):
            w24 |= units[:, i] << (3 * i)
        q = np.stack([(w24 >> (8 * j)) & 0xFF for j in range(3)], axis=1)
        return q.reshape(kn // 8 * 3, n).astype(np.uint8)
    raise NotImplementedError(f"{w_bits} bit is not implemented yet.")


def pack_codes_reference_loops(u: np.ndarray, w_bits: int) -> np.ndarray:
    """The same packing written as the reference's row loop (llama/qlinear.py:86-116).

    Slow; used on small inputs to cross-check `pack_codes`.
    """
    intweight = u.astype(np.uint8)
    q = np.zeros((intweight.shape[0] // 8 * w_bits, intweight.shape[1]), dtype=np.uint8)
    i = row = 0
    if w_bits in (2, 4, 8):
        while row < q.shape[0]:
            for j in range(i, i + 8 // w_bits):
                q[row] |= intweight[j] << (w_bits * (j - i))
            i += 8 // w_bits
            row += 1
    elif w_bits == 3:
        while row < q.shape[0]:
            for j in range(i, i + 2):
                q[row] |= intweight[j] << (3 * (j - i))
            i += 2
            q[row] |= intweight[i] << 6
            row += 1
            q[row] |= (intweight[i] >> 2) & 1
            i += 1
            for j in range(i, i + 2):
                q[row] |= intweight[j] << (3 * (j - i) + 1)
            i += 2
            q[row] |= intweight[i] << 7
            row += 1
            q[row] |= (intweight[i] >> 1) & 0x3
            i += 1
            for j in range(i, i + 2):
                q[row] |= intweight[j] << (3 * (j - i) + 2)
            i += 2
            row += 1
    else:
        raise NotImplementedError(f"{w_bits} bit is not implemented yet.")
    return q


def unpack_codes(qweight: np.ndarray, w_bits: int) -> np.ndarray:
    """Inverse of pack_codes: (Kn/8*b, N) uint8 -> codes (Kn, N) uint8.

    llama/qlinear.py:122-150 (torch shift tables) and the kernels' decode,
    csrc/quant_cuda_kernel.cu:811-829 (4-bit), 649-667 (3-bit).
    """
    rows, n = qweight.shape
    q = qweight.astype(np.uint32)
    if w_bits in (2, 4, 8):
        per = 8 // w_bits
        u = np.empty((rows * per, n), dtype=np.uint8)
        for t in range(per):
            u[t::per] = (q >> (w_bits * t)) & (2 ** w_bits - 1)
        return u
    if w_bits == 3:
        assert rows % 3 == 0
        q = q.reshape(rows // 3, 3, n)
        w24 = q[:, 0] | (q[:, 1] << 8) | (q[:, 2] << 16)
        u = np.stack([(w24 >> (3 * i)) & 7 for i in range(8)], axis=1)
        return u.reshape(rows // 3 * 8, n).astype(np.uint8)
    raise NotImplementedError(f"{w_bits} bit is not implemented yet.")


def unpack_codes_kernel_decode(qweight: np.ndarray) -> np.ndarray:
    """3-bit decode written as the CUDA kernel does it, byte by byte.

    csrc/quant_cuda_kernel.cu:649-667.  Cross-check for `unpack_codes(…, 3)`.
    """
    rows, n = qweight.shape
    q = qweight.astype(np.uint32).reshape(rows // 3, 3, n)
    q1, q2, q3 = q[:, 0], q[:, 1], q[:, 2]
    v = [q1 & 7, (q1 >> 3) & 7, ((q1 >> 6) | ((q2 << 2) & 4)) & 7, (q2 >> 1) & 7,
         (q2 >> 4) & 7, ((q2 >> 7) | ((q3 << 1) & 6)) & 7, (q3 >> 2) & 7, (q3 >> 5) & 7]
    return np.stack(v, axis=1).reshape(rows // 3 * 8, n).astype(np.uint8)


# --------------------------------------------------------------------------- pack / unpack

def pack(weight: np.ndarray, cherry_indices, w_bits: int, group_size: int) -> dict:
    """QuantLinear.pack: dense (N, K) weight + cherry columns -> the four packed buffers.

    llama/qlinear.py:67-118.  `weight` keeps its dtype (fp16 in pack.py:17).
    """
    n, k = weight.shape
    g = group_size if group_size != -1 else k
    idx = np.sort(np.asarray(cherry_indices, dtype=np.int64))
    nidx = normal_indices(k, idx)
    cherry_weight = np.ascontiguousarray(weight.T[idx]).astype(F16)
    normal_weight = weight[:, nidx]
    scales = get_scaling_factors(normal_weight, w_bits, g).astype(F16)
    s_full = expand_scales(scales, g, normal_weight.shape[1])
    q = quantize(normal_weight, s_full.astype(weight.dtype) if weight.dtype != F16 else s_full, w_bits)
    u = (q.T - iinfo(w_bits)[0]).astype(np.uint8)
    return {
        "cherry_indices": idx.astype(np.int16),
        "cherry_weight": cherry_weight,
        "qweight": pack_codes(np.ascontiguousarray(u), w_bits),
        "scales": np.ascontiguousarray(scales.T),
    }


def unpack(packed: dict, w_bits: int, group_size: int, in_features: int) -> np.ndarray:
    """QuantLinear.unpack: dense (N, K) fp16 weight.  llama/qlinear.py:120-162."""
    g = group_size if group_size != -1 else in_features
    qweight, scales = packed["qweight"], packed["scales"]
    idx = packed["cherry_indices"].astype(np.int64)
    n = qweight.shape[1]
    u = unpack_codes(qweight, w_bits).T  # (N, Kn)
    q = u.astype(np.int8) + np.int8(iinfo(w_bits)[0]) if w_bits < 8 else u.astype(np.int16) + iinfo(w_bits)[0]
    s = expand_scales(np.ascontiguousarray(scales.T), g, q.shape[1])
    deq = dequantize(q, s)
    w = np.zeros((n, in_features), dtype=F16)
    w[:, normal_indices(in_features, idx)] = deq
    w[:, idx] = packed["cherry_weight"].T
    return w


def adjust_weight(weight: np.ndarray, cherry_indices, w_bits: int, group_size: int) -> np.ndarray:
    """Fake-quantised inference weight.  llama/cherry_linear.py:77-99 (ste=False)."""
    n, k = weight.shape
    g = group_size if group_size != -1 else k
    nidx = normal_indices(k, cherry_indices)
    qw = weight[:, nidx]
    s = expand_scales(get_scaling_factors(qw, w_bits, g), g, qw.shape[1])
    out = weight.copy()
    out[:, nidx] = transform(qw, s, w_bits)
    return out


# --------------------------------------------------------------------------- forward

def dequant_forward(x: np.ndarray, w_dense: np.ndarray, bias=None, acc=np.float64) -> np.ndarray:
    """Dequantised forward: y = x @ W^T (+ bias), one rounding to fp16.

    llama/qlinear.py:194-198.  torch's CPU fp16 `linear` leaves the summation order
    unspecified; the oracle accumulates exactly-converted operands in `acc`.
    """
    y = x.astype(acc) @ w_dense.astype(acc).T
    if bias is not None:
        y = y.astype(F16).astype(acc) + bias.astype(acc)
    return y.astype(x.dtype)


def fused_forward(x, packed, w_bits, group_size, out_init=None, acc=np.float64):
    """Entry-point contract of vecquant{3,4}matmul_cherryq, summed in `acc`:

    mul[b,n] += sum_k (u[k,n]-c_b) s[k//G,n] x[b,normal[k]] + sum_c cw[c,n] x[b,idx[c]]
    csrc/quant_cuda_kernel.cu:718-835 (4-bit), 558-672 (3-bit), un-rounded weights.
    """
    k = x.shape[1]
    g = group_size if group_size != -1 else k
    idx = packed["cherry_indices"].astype(np.int64)
    nidx = normal_indices(k, idx)
    u = unpack_codes(packed["qweight"], w_bits).astype(acc)
    c_b = 2 ** (w_bits - 1) - 0.5
    s = np.repeat(packed["scales"].astype(acc), g, axis=0)[: u.shape[0]]
    wn = (u - c_b) * s
    y = x[:, nidx].astype(acc) @ wn + x[:, idx].astype(acc) @ packed["cherry_weight"].astype(acc)
    if out_init is not None:
        y = y + out_init.astype(acc)
    return y


def fused_reference_order(x, packed, w_bits, group_size, io=F16):
    """The CUDA kernels' own evaluation order for group sizes that are multiples of 128:
    per 128 normal positions an fp32 sum of (u-c)*x, times fp32(scale), rounded to the
    I/O type, then summed in the I/O type (block order 0.., cherries last).

    csrc/quant_cuda_kernel.cu:797-834 and 738-762.  The device adds the blocks with
    atomics in arbitrary order; this function uses ascending order.
    """
    b, k = x.shape
    idx = packed["cherry_indices"].astype(np.int64)
    nidx = normal_indices(k, idx)
    u = unpack_codes(packed["qweight"], w_bits).astype(F32)
    kn, n = u.shape
    c_b = F32(2 ** (w_bits - 1) - 0.5)
    ng = math.ceil(kn / group_size)
    xn = x[:, nidx].astype(F32)
    out = np.zeros((b, n), dtype=io)
    for blk in range(math.ceil(kn / 128)):
        gi = blk // (group_size // 128)
        factor = packed["scales"][gi].astype(F32) if gi < ng else np.zeros(n, F32)
        lo, hi = blk * 128, min(blk * 128 + 128, kn)
        res = np.zeros((b, n), dtype=F32)
        for j in range(lo, hi):
            res += (u[j] - c_b)[None, :] * xn[:, j:j + 1]
        out = (out.astype(F32) + (factor[None, :] * res).astype(io).astype(F32)).astype(io)
    for blk in range(math.ceil(idx.shape[0] / 128)):
        res = np.zeros((b, n), dtype=F32)
        for c in range(blk * 128, min(blk * 128 + 128, idx.shape[0])):
            res += packed["cherry_weight"][c].astype(F32)[None, :] * x[:, idx[c]].astype(F32)[:, None]
        out = (out.astype(F32) + res.astype(io).astype(F32)).astype(io)
    return out


def dequantize_normal(qweight, scales_f32, w_bits, height, cherry_size, group_size):
    """Dense fp32 dequant of the compacted normal part, out[k, n] = (u - c_b) * s[k//G, n].

    Intended semantics of Dequantize{3,4}Normal, csrc/quant_cuda_kernel.cu:838-1010
    (the 4-bit launcher there mis-indexes rows with the 3-bit block height, :934,:964;
    the oracle states the evident intent, identical to the 3-bit kernel's).
    """
    u = unpack_codes(qweight, w_bits).astype(F32)
    kn = height - cherry_size
    assert u.shape[0] == kn
    c_b = F32(2 ** (w_bits - 1) - 0.5)
    s = np.repeat(scales_f32.astype(F32), group_size, axis=0)[:kn]
    return (u - c_b) * s


# --------------------------------------------------------------------------- synthetic layers

def synthetic_layer(in_features, out_features, w_bits, group_size=128, seed=0,
                    cherry_fraction=1 / 256, outlier_fraction=0.01, outlier_gain=10.0):
    """Seeded CherryLinear in the reference buffer schema.

    W ~ N(0, 0.02^2), 1 % of the entries scaled x10, cast to fp16 (as pack.py:17 loads
    fp16 weights).  Cherry columns: the C input channels with the largest max|w|, sorted.
    Returns (weight_fp16, packed dict).
    """
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((out_features, in_features), dtype=F32) * F32(0.02)
    mask = rng.random((out_features, in_features), dtype=F32) < outlier_fraction
    w = np.where(mask, w * F32(outlier_gain), w).astype(F16)
    c = num_cherries(in_features, cherry_fraction)
    score = np.max(np.abs(w), axis=0).astype(F32)
    idx = np.sort(np.argsort(-score, kind="stable")[:c])
    return w, pack(w, idx, w_bits, group_size)


def synthetic_packed_fast(in_features, out_features, w_bits, group_size=128, seed=0,
                          cherry_fraction=1 / 256):
    """Random packed buffers of valid shape (uniform codes, plausible scales) without
    going through quantisation; for large-shape property tests and benchmarks."""
    rng = np.random.default_rng(seed)
    shapes = buffer_shapes(w_bits, group_size, in_features, out_features, cherry_fraction)
    c = shapes["cherry_indices"][0][0]
    idx = np.sort(rng.choice(in_features, size=c, replace=False)).astype(np.int16)
    qweight = rng.integers(0, 256, size=shapes["qweight"][0], dtype=np.uint8)
    scales = (rng.random(shapes["scales"][0], dtype=F32) * F32(0.01) + F32(0.005)).astype(F16)
    cw = (rng.standard_normal(shapes["cherry_weight"][0], dtype=F32) * F32(0.1)).astype(F16)
    return {"cherry_indices": idx, "cherry_weight": cw, "qweight": qweight, "scales": scales}


# --------------------------------------------------------------------------- weight stream
# The load-time repack of include/cherryq.h (cherryq_prepack_f16) has no counterpart in the
# reference: it is this build's own rearrangement of the reference buffers.  What pins it is
# that it is a bijection of them: stream_unpack(stream_pack(p)) == p for every buffer, and the
# device kernels must produce these very bytes.  Codes are read from `qweight` with unpack_codes
# (llama/qlinear.py:120-150), positions are the compacted normal positions of
# csrc/quant_cuda_kernel.cu:785-795.

def _align256(v):
    return (v + 255) & ~255


def stream_geometry(w_bits, in_features, out_features, num_cherries):
    kn = in_features - num_cherries
    ng = -(-kn // 128)
    cp = (num_cherries + 31) & ~31
    off_cherry = _align256(ng * 32)
    off_units = off_cherry + _align256(num_cherries * 32)
    unit_bytes = 1024 if w_bits == 4 else 768
    return dict(kn=kn, ng=ng, cp=cp, ntiles=-(-out_features // 16), off_cherry=off_cherry, off_units=off_units,
                unit_bytes=unit_bytes, record_bytes=off_units + ng * unit_bytes,
                knp512=(ng * 128 + 511) & ~511, hdr_bytes=_align256(((ng * 128 + 511) & ~511) + 2 * cp))


def _stream_slot(w_bits):
    """For code q (0..31) of a lane: (dword, bit) of its field, dword 3 = the two 3-bit codes
    spread over bit 15 + 16 h of dwords 0..2."""
    slots = []
    for q in range(32):
        if w_bits == 4:
            j, r = q >> 3, q & 7
            slots.append((2 * (j & 1) + (r >> 2), 4 * ([0, 4, 2, 6][r & 3] + (j >> 1))))
        else:
            h = q & 1
            if q < 24:
                r, m = q & 7, q >> 3
                if r < 6:
                    slots.append((r >> 1, 16 * h + 3 * m))
                elif q < 16:
                    slots.append((0, 16 * h + 3 * (m + 3)))
                else:
                    slots.append((3, 16 * h))
            else:
                slots.append((1 + ((q & 3) >> 1), 16 * h + 3 * (3 if q < 28 else 4)))
    return slots


def stream_pack(packed, w_bits, group_size, in_features):
    """Reference buffers -> weight stream (uint8 array), as cherryq_prepack_f16 lays it out."""
    qweight, scales = packed["qweight"], packed["scales"]
    cw, idx = packed["cherry_weight"], packed["cherry_indices"].astype(np.int64)
    n = qweight.shape[1]
    c = idx.shape[0]
    g = stream_geometry(w_bits, in_features, n, c)
    kn, ng = g["kn"], g["ng"]
    assert group_size % 128 == 0
    out = np.zeros(g["hdr_bytes"] + g["ntiles"] * g["record_bytes"], dtype=np.uint8)
    # header: low(k) per compacted position, lane-transposed per block of 512; then cherry columns
    k = np.arange(g["knp512"])
    low = np.where(k < kn, gather_offset(np.minimum(k, max(kn - 1, 0)), idx), c).astype(np.uint8)
    blk, l, j = k >> 9, (k >> 3) & 63, k & 7           # stored index -> position blk*512 + 64 j + l
    out[:g["knp512"]] = low[blk * 512 + 64 * j + l]
    cidx = np.full(g["cp"], in_features, dtype=np.uint16)
    cidx[:c] = idx
    out[g["knp512"]:g["knp512"] + 2 * g["cp"]] = cidx.view(np.uint8)
    codes = np.zeros((ng * 128, g["ntiles"] * 16), dtype=np.uint32)
    codes[:kn, :n] = unpack_codes(qweight, w_bits)
    sc = np.zeros((ng, g["ntiles"] * 16), dtype=np.float16)
    sc[:, :n] = scales[(np.arange(ng) * 128) // group_size]
    cwp = np.zeros((c, g["ntiles"] * 16), dtype=np.float16)
    cwp[:, :n] = cw
    slots = _stream_slot(w_bits)
    dw = w_bits
    # units: [tile][g][lane = kq*16 + nn][dword]
    cu = codes.reshape(ng, 4, 32, g["ntiles"], 16)       # g, kq, q, tile, nn
    words = np.zeros((g["ntiles"], ng, 4, 16, 4), dtype=np.uint32)
    for q, (d, bit) in enumerate(slots):
        v = cu[:, :, q].transpose(2, 0, 1, 3)             # tile, g, kq, nn
        if d < 3 or w_bits == 4:
            words[..., d] |= v << bit
        else:
            for b in range(3):
                words[..., b] |= ((v >> b) & 1) << (bit + 15)
    rec = out[g["hdr_bytes"]:].reshape(g["ntiles"], g["record_bytes"])
    rec[:, :ng * 32] = sc.reshape(ng, g["ntiles"], 16).transpose(1, 0, 2).reshape(g["ntiles"], -1).view(np.uint8)
    if c:
        # piece (lg, nn): cherry rows 8 lg .. 8 lg + 7 of column nn
        cp_ = cwp.reshape(c // 8, 8, g["ntiles"], 16).transpose(2, 0, 3, 1)   # tile, lg, nn, e
        rec[:, g["off_cherry"]:g["off_cherry"] + c * 32] = np.ascontiguousarray(cp_).reshape(g["ntiles"], -1).view(np.uint8)
    rec[:, g["off_units"]:] = np.ascontiguousarray(words[..., :dw]).reshape(g["ntiles"], -1).view(np.uint8)
    return out


def stream_unpack(stream, w_bits, group_size, in_features, out_features, num_cherries):
    """Inverse of stream_pack: the reference buffers back, bit for bit."""
    g = stream_geometry(w_bits, in_features, out_features, num_cherries)
    kn, ng, n, c = g["kn"], g["ng"], out_features, num_cherries
    cidx = stream[g["knp512"]:g["knp512"] + 2 * g["cp"]].view(np.uint16)[:c].astype(np.int16)
    rec = stream[g["hdr_bytes"]:].reshape(g["ntiles"], g["record_bytes"])
    sc = rec[:, :ng * 32].copy().view(np.float16).reshape(g["ntiles"], ng, 16).transpose(1, 0, 2).reshape(ng, -1)[:, :n]
    ngr = -(-kn // group_size)
    scales = sc[(np.arange(ngr) * group_size) // 128]
    cw = np.zeros((c, n), dtype=np.float16)
    if c:
        cp_ = rec[:, g["off_cherry"]:g["off_cherry"] + c * 32].copy().view(np.float16).reshape(g["ntiles"], c // 8, 16, 8)
        cw = cp_.transpose(1, 3, 0, 2).reshape(c, -1)[:, :n]
    dw = w_bits
    words = rec[:, g["off_units"]:].copy().view(np.uint32).reshape(g["ntiles"], ng, 4, 16, dw)
    codes = np.zeros((ng, 4, 32, g["ntiles"], 16), dtype=np.uint8)
    for q, (d, bit) in enumerate(_stream_slot(w_bits)):
        if d < 3 or w_bits == 4:
            v = (words[..., d] >> bit) & (2 ** w_bits - 1)
        else:
            v = sum((((words[..., b] >> (bit + 15)) & 1) << b) for b in range(3))
        codes[:, :, q] = v.transpose(1, 2, 0, 3)
    codes = codes.reshape(ng * 128, -1)[:kn, :n]
    return {"cherry_indices": cidx, "cherry_weight": np.ascontiguousarray(cw), "qweight": pack_codes(codes, w_bits),
            "scales": np.ascontiguousarray(scales)}


def rel_l2(a, b) -> float:
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))
