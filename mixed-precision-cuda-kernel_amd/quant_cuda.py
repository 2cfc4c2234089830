"""`quant_cuda` for MI355X: the reference extension's four entry points over libcherryq.

Drop-in for the pybind11 module built from csrc/quant_cuda.cpp:72-77 of the reference:

    vecquant3matmul_cherryq(vec, qweight, cherry_weight, cherry_indices, scaling_factors, mul, group_size, fp16)
    vecquant4matmul_cherryq(vec, qweight, cherry_weight, cherry_indices, scaling_factors, mul, group_size)
    Dequantize3Normal(qweight, scaling_factors, out, height, cherry_size, group_size)
    Dequantize4Normal(qweight, scaling_factors, out, height, cherry_size, group_size)

Same positional arguments, same in-place accumulate into `mul`, nothing returned.  The work is
done by hand-written HIP kernels in libcherryq.so (C ABI: include/cherryq.h), reached through
ctypes with raw device pointers; torch only supplies memory and the current stream.  There is no
CPU or eager fallback: importing this module without the built library raises, and so does any
call with tensors that are not on a GPU.

Differences from the reference, all on the side of failing loudly (the reference launches on
the legacy default stream without checking anything, csrc/quant_cuda_kernel.cu:140,699):
kernels run on torch's current stream; dtype / device / shape / contiguity mismatches raise
RuntimeError; group sizes the kernels cannot honour raise instead of silently doing nothing
(csrc/quant_cuda_kernel.cu:139-179).
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
_LIB_PATH = Path(os.environ.get("CHERRYQ_LIB", _HERE / "libcherryq.so"))

if not _LIB_PATH.exists():
    raise ImportError(
        f"quant_cuda: {_LIB_PATH} is not built. Run `python {_HERE / 'build.py'}` "
        "(hipcc, --offload-arch=gfx950); there is no fallback implementation.")

_lib = ctypes.CDLL(str(_LIB_PATH))

_vp, _int, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_MATMUL_ARGS = [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _vp, _sz, _vp, _sz, _vp]
for _name in ("cherryq_vecquant4matmul_f16", "cherryq_vecquant3matmul_f16", "cherryq_vecquant3matmul_f32"):
    getattr(_lib, _name).argtypes = _MATMUL_ARGS
    getattr(_lib, _name).restype = _int
for _name in ("cherryq_dequantize3_normal_f32", "cherryq_dequantize4_normal_f32"):
    getattr(_lib, _name).argtypes = [_vp, _vp, _vp, _int, _int, _int, _int, _vp]
    getattr(_lib, _name).restype = _int
_lib.cherryq_unpack_f16.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]
_lib.cherryq_unpack_f16.restype = _int
_lib.cherryq_pack_f16.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]
_lib.cherryq_pack_f16.restype = _int
for _name in ("cherryq_fake_quant_f16", "cherryq_fake_quant_f32"):
    getattr(_lib, _name).argtypes = [_int, _vp, _vp, _vp, _int, _int, _int, _int, _int, _vp]
    getattr(_lib, _name).restype = _int
_lib.cherryq_vecquant_matmul_f16_static.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _vp]
_lib.cherryq_vecquant_matmul_f16_static.restype = _int
_lib.cherryq_set_force_generic.argtypes = [_int]
_lib.cherryq_set_force_generic.restype = None
_lib.cherryq_prepacked_scratch_bytes.argtypes = [_int, _int, _int, _int, _int]
_lib.cherryq_prepacked_scratch_bytes.restype = _sz
_lib.cherryq_matmul_prepacked_f16.argtypes = [_int, _vp, _vp, _sz, _vp, _int, _int, _int, _int, _int, _vp, _sz, _vp]
_lib.cherryq_matmul_prepacked_f16.restype = _int
_lib.cherryq_prepack_bytes.argtypes = [_int, _int, _int, _int]
_lib.cherryq_prepack_bytes.restype = _sz
_lib.cherryq_prepack_supported.argtypes = [_int, _int, _int, _int, _int, _int]
_lib.cherryq_prepack_supported.restype = _int
_lib.cherryq_prepack_recommended.argtypes = [_int, _int, _int, _int, _int]
_lib.cherryq_prepack_recommended.restype = _int
_lib.cherryq_prepack_rows_recommended.argtypes = [_int, _int, _int, _int, _int, _int]
_lib.cherryq_prepack_rows_recommended.restype = _int
_lib.cherryq_prepack_f16.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _sz, _int, _int, _int, _int, _vp]
_lib.cherryq_prepack_f16.restype = _int
_lib.cherryq_unprepack_f16.argtypes = [_int, _vp, _sz, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]
_lib.cherryq_unprepack_f16.restype = _int
_lib.cherryq_matvec_prepacked_f16.argtypes = [_int, _vp, _vp, _sz, _vp, _int, _int, _int, _int, _int, _vp]
_lib.cherryq_matvec_prepacked_f16.restype = _int
_lib.cherryq_workspace_bytes.argtypes = [_int, _int, _int, _int]
_lib.cherryq_workspace_bytes.restype = _sz
_lib.cherryq_scratch_bytes.argtypes = [_int, _int, _int, _int]
_lib.cherryq_scratch_bytes.restype = _sz
_lib.cherryq_scratch_bytes_f32.argtypes = [_int, _int, _int, _int]
_lib.cherryq_scratch_bytes_f32.restype = _sz
_lib.cherryq_status_string.argtypes = [_int]
_lib.cherryq_status_string.restype = ctypes.c_char_p
_lib.cherryq_version.restype = _int

LIBRARY_PATH = str(_LIB_PATH)


def _fail(status: int, what: str):
    raise RuntimeError(f"{what}: {_lib.cherryq_status_string(status).decode()} (status {status})")


def _check(t: torch.Tensor, name: str, dtype, ndim: int, device=None):
    # one compound test for the tensor that is fine (this runs six times per call); the
    # individual tests below only word the error
    if (isinstance(t, torch.Tensor) and t.dtype == dtype and t.dim() == ndim and t.is_cuda
            and (device is None or t.device == device) and t.is_contiguous()):
        return
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise RuntimeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if t.dim() != ndim:
        raise RuntimeError(f"{name}: expected {ndim} dimensions, got {tuple(t.shape)}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on a GPU (got {t.device}); there is no CPU path")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name} is on {t.device}, expected {device}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


# Per (device, stream): a zero-initialised workspace (the kernels leave it all zero after every
# call, so it is reusable as is) and an uninitialised scratch buffer for the batched path.  Both
# grow on demand, at least doubling.  An outgrown buffer is kept alive rather than freed: a HIP
# graph captured earlier on that stream may still hold its address (doubling bounds what is kept
# to the size of the live buffer).
_workspaces: dict = {}
_scratches: dict = {}
_outgrown: list = []
_sizes: dict = {}  # (batch, in, out, cherries, dtype) -> (workspace bytes, scratch bytes) as the library reports them


def _grown(table: dict, key, nbytes: int, floor: int, alloc, device) -> torch.Tensor:
    buf = table.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _outgrown.append(buf)
            nbytes = max(nbytes, 2 * buf.numel())
        buf = alloc(max(nbytes, floor), dtype=torch.uint8, device=device)
        table[key] = buf
    return buf


def _workspace(device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
    return _grown(_workspaces, (device.index, stream), nbytes, 1 << 18, torch.zeros, device)


def _scratch(device: torch.device, stream: int, nbytes: int):
    if nbytes == 0:
        return None
    return _grown(_scratches, (device.index, stream), nbytes, 1, torch.empty, device)


# torch's current stream as a raw handle.  The private accessor costs a tenth of building a
# torch.cuda.Stream object per call (2.8 us, a quarter of a whole call's host time); the public
# way is the fallback where it does not exist.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device_index: int) -> int:
    if _raw_stream is not None:
        return _raw_stream(device_index)
    return torch.cuda.current_stream(device_index).cuda_stream


def _ptr(t: torch.Tensor):
    return t.data_ptr() if t.numel() else None


def _matmul(fn, what, vec, qweight, cherry_weight, cherry_indices, scales, mul, group_size, w_bits,
            io_dtype, idx_dtype, accumulate=True):
    _check(vec, "vec", io_dtype, 2)
    dev = vec.device
    _check(qweight, "qweight", torch.uint8, 2, dev)
    _check(cherry_weight, "cherry_weight", io_dtype, 2, dev)
    _check(cherry_indices, "cherry_indices", idx_dtype, 1, dev)
    _check(scales, "scaling_factors", io_dtype, 2, dev)
    _check(mul, "mul", io_dtype, 2, dev)
    batch, k = vec.shape
    n = qweight.shape[1]
    c = cherry_indices.shape[0]
    group_size = int(group_size)
    kn = k - c
    if qweight.shape[0] * 8 != kn * w_bits:
        raise RuntimeError(f"qweight has {qweight.shape[0]} rows, expected {(kn // 8) * w_bits} "
                           f"for in_features={k}, num_cherries={c}, w_bits={w_bits}")
    if tuple(cherry_weight.shape) != (c, n):
        raise RuntimeError(f"cherry_weight shape {tuple(cherry_weight.shape)} != {(c, n)}")
    if group_size <= 0:
        raise RuntimeError(f"{what}: group_size must be positive, got {group_size}")
    ng = -(-kn // group_size)
    if tuple(scales.shape) != (ng, n):
        raise RuntimeError(f"scaling_factors shape {tuple(scales.shape)} != {(ng, n)}")
    if tuple(mul.shape) != (batch, n):
        raise RuntimeError(f"mul shape {tuple(mul.shape)} != {(batch, n)}")
    if batch == 0:
        return
    if torch.cuda.current_device() != dev.index:
        with torch.cuda.device(dev):
            return _matmul(fn, what, vec, qweight, cherry_weight, cherry_indices, scales, mul, group_size,
                           w_bits, io_dtype, idx_dtype, accumulate)
    stream = _current_stream(dev.index)
    sizes = _sizes.get((batch, k, n, c, io_dtype))
    if sizes is None:
        sizes = (_lib.cherryq_workspace_bytes(batch, k, n, c),
                 _lib.cherryq_scratch_bytes_f32(batch, k, n, c) if io_dtype == torch.float32
                 else _lib.cherryq_scratch_bytes(batch, k, n, c) if batch > 1 else 0)
        if len(_sizes) < 4096:
            _sizes[(batch, k, n, c, io_dtype)] = sizes
    ws = _workspace(dev, stream, sizes[0])
    sc = _scratch(dev, stream, sizes[1])
    rc = fn(_ptr(vec), _ptr(qweight), _ptr(cherry_weight), _ptr(cherry_indices), _ptr(scales), _ptr(mul),
            batch, k, n, c, group_size, 1 if accumulate else 0, ws.data_ptr(), ws.numel(),
            sc.data_ptr() if sc is not None else None, sc.numel() if sc is not None else 0, stream)
    if rc != 0:
        _fail(rc, what)


def vecquant4matmul_cherryq(vec, qweight, cherry_weight, cherry_indices, scaling_factors, mul, group_size):
    """mul += vec @ W^T for 4-bit packed W (reference: csrc/quant_cuda.cpp:56-69)."""
    if int(group_size) < 128:
        raise RuntimeError("`group_size` must be multiple of 128")  # csrc/quant_cuda_kernel.cu:684
    _matmul(_lib.cherryq_vecquant4matmul_f16, "vecquant4matmul_cherryq", vec, qweight, cherry_weight,
            cherry_indices, scaling_factors, mul, group_size, 4, torch.float16, torch.int16)


def vecquant3matmul_cherryq(vec, qweight, cherry_weight, cherry_indices, scaling_factors, mul, group_size,
                            fp16):
    """mul += vec @ W^T for 3-bit packed W (reference: csrc/quant_cuda.cpp:41-54).

    fp16=True: fp16 tensors, int16 indices.  fp16=False: fp32 tensors, int32 indices
    (the call shape of benchmark_speed.py:20-32)."""
    if fp16:
        _matmul(_lib.cherryq_vecquant3matmul_f16, "vecquant3matmul_cherryq", vec, qweight, cherry_weight,
                cherry_indices, scaling_factors, mul, group_size, 3, torch.float16, torch.int16)
    else:
        _matmul(_lib.cherryq_vecquant3matmul_f32, "vecquant3matmul_cherryq", vec, qweight, cherry_weight,
                cherry_indices, scaling_factors, mul, group_size, 3, torch.float32, torch.int32)


def matmul_cherryq(w_bits, vec, qweight, cherry_weight, cherry_indices, scaling_factors, out, group_size,
                   accumulate=False):
    """fp16 fused matmul that can overwrite `out` instead of accumulating into it, which spares
    the caller the zero-fill the reference needs before every call (llama/qlinear.py:177).
    No counterpart in the reference extension."""
    if w_bits == 4:
        if int(group_size) < 128:
            raise RuntimeError("`group_size` must be multiple of 128")
        fn = _lib.cherryq_vecquant4matmul_f16
    elif w_bits == 3:
        fn = _lib.cherryq_vecquant3matmul_f16
    else:
        raise NotImplementedError(f"{w_bits} bit kernel is not implemented yet.")
    _matmul(fn, f"matmul_cherryq[{w_bits}bit]", vec, qweight, cherry_weight, cherry_indices, scaling_factors,
            out, group_size, w_bits, torch.float16, torch.int16, accumulate=accumulate)


def force_generic(on: bool) -> None:
    """Test hook: route every fused call through the library's general kernel (the tests compare it
    with the specialised ones)."""
    _lib.cherryq_set_force_generic(1 if on else 0)


def matmul_cherryq_static(w_bits, vec, qweight, cherry_weight, cherry_indices, scaling_factors, out, group_size,
                          accumulate=False):
    """matmul_cherryq for 1 to 4 rows without any device allocation or workspace of the caller's:
    the split-K accumulators live in a fixed 1 MiB array inside the library (so batch *
    out_features <= 131072), shared by all calls on a GPU -- calls on different streams of one GPU
    must not overlap.  For code under graph capture and loops that may not allocate."""
    _check(vec, "vec", torch.float16, 2)
    dev = vec.device
    _check(qweight, "qweight", torch.uint8, 2, dev)
    _check(cherry_weight, "cherry_weight", torch.float16, 2, dev)
    _check(cherry_indices, "cherry_indices", torch.int16, 1, dev)
    _check(scaling_factors, "scaling_factors", torch.float16, 2, dev)
    _check(out, "out", torch.float16, 2, dev)
    b, k = vec.shape
    n, c = qweight.shape[1], cherry_indices.shape[0]
    kn = k - c
    if qweight.shape[0] * 8 != kn * w_bits or cherry_weight.shape != (c, n) or tuple(out.shape) != (b, n):
        raise RuntimeError("matmul_cherryq_static: buffer shapes do not match")
    if int(group_size) <= 0 or tuple(scaling_factors.shape) != (-(-kn // int(group_size)), n):
        raise RuntimeError(f"scaling_factors shape {tuple(scaling_factors.shape)} does not match group_size={group_size}")
    with torch.cuda.device(dev):
        rc = _lib.cherryq_vecquant_matmul_f16_static(int(w_bits), _ptr(vec), _ptr(qweight), _ptr(cherry_weight),
                                                     _ptr(cherry_indices), _ptr(scaling_factors), _ptr(out), b, k, n, c,
                                                     int(group_size), 1 if accumulate else 0,
                                                     _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "matmul_cherryq_static")


def _dequantize_normal(fn, what, w_bits, qweight, scaling_factors, out, height, cherry_size, group_size):
    _check(qweight, "qweight", torch.uint8, 2)
    dev = qweight.device
    _check(scaling_factors, "scaling_factors", torch.float32, 2, dev)
    _check(out, "out", torch.float32, 2, dev)
    height, cherry_size, group_size = int(height), int(cherry_size), int(group_size)
    n = qweight.shape[1]
    kn = height - cherry_size
    if qweight.shape[0] * 8 != kn * w_bits:
        raise RuntimeError(f"qweight has {qweight.shape[0]} rows, expected {(kn // 8) * w_bits}")
    if group_size <= 0 or tuple(scaling_factors.shape) != (-(-kn // group_size), n):
        raise RuntimeError(f"scaling_factors shape {tuple(scaling_factors.shape)} does not match "
                           f"group_size={group_size}")
    if out.shape[1] != n or out.shape[0] < kn:
        raise RuntimeError(f"out shape {tuple(out.shape)} cannot hold ({kn}, {n})")
    with torch.cuda.device(dev):
        rc = fn(_ptr(qweight), _ptr(scaling_factors), _ptr(out), height, n, cherry_size, group_size,
                _current_stream(dev.index))
    if rc != 0:
        _fail(rc, what)


def Dequantize3Normal(qweight, scaling_factors, out, height, cherry_size, group_size):
    """out[k, n] = (code - 3.5) * scale for the compacted normal part (reference:
    csrc/quant_cuda_kernel.cu:838-922)."""
    _dequantize_normal(_lib.cherryq_dequantize3_normal_f32, "Dequantize3Normal", 3, qweight, scaling_factors,
                       out, height, cherry_size, group_size)


def Dequantize4Normal(qweight, scaling_factors, out, height, cherry_size, group_size):
    """out[k, n] = (code - 7.5) * scale for the compacted normal part.  The reference's
    launcher (csrc/quant_cuda_kernel.cu:925-1010) walks the rows with the 3-bit block height
    and leaves part of `out` unwritten; this one writes all Kn rows."""
    _dequantize_normal(_lib.cherryq_dequantize4_normal_f32, "Dequantize4Normal", 4, qweight, scaling_factors,
                       out, height, cherry_size, group_size)


def unpack_cherryq(w_bits, qweight, cherry_weight, cherry_indices, scaling_factors, in_features, group_size):
    """Dense (out_features, in_features) fp16 weight, bit for bit what QuantLinear.unpack()
    computes (llama/qlinear.py:120-162), produced on the GPU."""
    _check(qweight, "qweight", torch.uint8, 2)
    dev = qweight.device
    _check(cherry_weight, "cherry_weight", torch.float16, 2, dev)
    _check(cherry_indices, "cherry_indices", torch.int16, 1, dev)
    _check(scaling_factors, "scaling_factors", torch.float16, 2, dev)
    n = qweight.shape[1]
    c = cherry_indices.shape[0]
    kn = int(in_features) - c
    if qweight.shape[0] * 8 != kn * w_bits:
        raise RuntimeError(f"qweight has {qweight.shape[0]} rows, expected {(kn // 8) * w_bits}")
    if tuple(scaling_factors.shape) != (-(-kn // int(group_size)), n):
        raise RuntimeError(f"scaling_factors shape {tuple(scaling_factors.shape)} does not match")
    dense = torch.empty((n, int(in_features)), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.cherryq_unpack_f16(w_bits, _ptr(qweight), _ptr(cherry_weight), _ptr(cherry_indices),
                                     _ptr(scaling_factors), dense.data_ptr(), int(in_features), n, c,
                                     int(group_size), _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "unpack_cherryq")
    return dense


def pack_cherryq(w_bits, weight, cherry_indices, group_size):
    """pack() on the GPU: dense fp16 `weight` (out, in) and the cherry channels (any order, any
    integer dtype) -> (cherry_indices int16 ascending, cherry_weight, qweight, scales) in the
    packed schema, bit for bit what QuantLinear.pack() computes on the host
    (llama/qlinear.py:67-118).  No counterpart in the reference extension."""
    _check(weight, "weight", torch.float16, 2)
    dev = weight.device
    if w_bits not in (3, 4):
        raise NotImplementedError(f"{w_bits} bit is not implemented yet.")
    n, k = weight.shape
    idx = cherry_indices.to(device=dev).sort().values
    c = idx.numel()
    if c and (int(idx[0]) < 0 or int(idx[-1]) >= k or bool((idx[1:] == idx[:-1]).any())):
        raise RuntimeError("cherry_indices must be distinct channels in [0, in_features)")
    idx = idx.to(torch.int16).contiguous()
    group_size = int(group_size) if int(group_size) != -1 else k
    kn = k - c
    if k % 8 or c % 8 or group_size <= 0:
        raise RuntimeError(f"pack_cherryq: in_features={k}, num_cherries={c}, group_size={group_size} not packable")
    qweight = torch.empty((kn // 8 * w_bits, n), dtype=torch.uint8, device=dev)
    scales = torch.empty((-(-kn // group_size), n), dtype=torch.float16, device=dev)
    cherry_weight = torch.empty((c, n), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.cherryq_pack_f16(w_bits, weight.data_ptr(), _ptr(idx), _ptr(qweight), _ptr(scales),
                                   _ptr(cherry_weight), k, n, c, group_size, _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "pack_cherryq")
    return idx, cherry_weight, qweight, scales


def prepack_supported(w_bits, batch, in_features, out_features, num_cherries, group_size) -> bool:
    """Whether the load-time repacked path takes this call shape (batch 1, group size a multiple
    of 128, at most 128 cherry channels and 16384 quantised input channels)."""
    return bool(_lib.cherryq_prepack_supported(int(w_bits), int(batch), int(in_features), int(out_features),
                                               int(num_cherries), int(group_size)))


def prepack_recommended(w_bits, in_features, out_features, num_cherries, group_size) -> bool:
    """Whether the matvec over the repacked stream measured faster on this GPU than the one over
    the checkpoint layout for this layer shape (what a loader asks before prepack_cherryq)."""
    return bool(_lib.cherryq_prepack_recommended(int(w_bits), int(in_features), int(out_features),
                                                 int(num_cherries), int(group_size)))


def prepacked_rows_recommended(w_bits, rows, in_features, out_features, num_cherries, group_size) -> bool:
    """Whether `rows` activation rows run faster over a layer's repacked stream than over its
    checkpoint buffers (for a caller that holds both): cherryq_prepack_rows_recommended.  Measured on
    MI355X, checkpoint layout / stream in us: 4096 -> 11008 4-bit 2 rows 9.1 / 6.6, 4 rows 11.3 / 7.4,
    8 rows 16.8 / 12.4; 4096 -> 4096 4 rows 8.1 / 5.6; 5120 -> 5120 3-bit 4 rows 7.9 / 7.5, 8 rows 13.7 / 11.9;
    5120 -> 13824 3-bit 4 rows 14.0 / 9.9, 8 rows 19.6 / 16.1; 8192 -> 28672 4 rows 32.9 / 23.1; 11008 -> 4096
    4-bit 2 rows 8.9 / 8.3, 4 rows 11.1 / 9.8, 8 rows 17.0 / 13.9, 16 rows 21.4 / 14.4; 28672 -> 8192 4-bit
    2 rows 27.4 / 30.2, 8 rows 36.1 / 30.4, 16 rows 41.3 / 32.6; 13824 -> 5120 3-bit 4 rows 13.6 / 16.3,
    8 rows 19.8 / 16.4."""
    return bool(_lib.cherryq_prepack_rows_recommended(int(w_bits), int(rows), int(in_features), int(out_features),
                                                      int(num_cherries), int(group_size)))


def prepacked_kernel_name(w_bits, in_features, out_features, num_cherries, rows=1) -> str:
    """The kernels matvec_prepacked_cherryq launches for a call of `rows` rows on this layer, as a profiler names them."""
    _lib.cherryq_matmul_prepacked_kernel_name.restype = ctypes.c_char_p
    return _lib.cherryq_matmul_prepacked_kernel_name(int(w_bits), int(rows), int(in_features), int(out_features),
                                                     int(num_cherries)).decode()


def prepack_cherryq(w_bits, qweight, cherry_weight, cherry_indices, scaling_factors, in_features, group_size):
    """The packed buffers of one layer rearranged, once, into the weight stream the batch-1 matvec
    of this GPU reads fastest (16 output columns' whole input range contiguous, codes placed
    where one mask makes them matrix-core operands).  Same information bit for bit;
    unprepack_cherryq is the exact inverse.  No counterpart in the reference extension."""
    _check(qweight, "qweight", torch.uint8, 2)
    dev = qweight.device
    _check(cherry_weight, "cherry_weight", torch.float16, 2, dev)
    _check(cherry_indices, "cherry_indices", torch.int16, 1, dev)
    _check(scaling_factors, "scaling_factors", torch.float16, 2, dev)
    k, n, c, g = int(in_features), qweight.shape[1], cherry_indices.shape[0], int(group_size)
    kn = k - c
    if qweight.shape[0] * 8 != kn * w_bits or tuple(cherry_weight.shape) != (c, n):
        raise RuntimeError("prepack_cherryq: buffer shapes do not match in_features / w_bits")
    if g <= 0 or tuple(scaling_factors.shape) != (-(-kn // g), n):
        raise RuntimeError(f"scaling_factors shape {tuple(scaling_factors.shape)} does not match group_size={g}")
    if not prepack_supported(w_bits, 1, k, n, c, g):
        raise RuntimeError(f"prepack_cherryq: shape not taken (w_bits={w_bits}, in={k}, out={n}, cherries={c}, group={g})")
    nbytes = _lib.cherryq_prepack_bytes(w_bits, k, n, c)
    stream = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.cherryq_prepack_f16(w_bits, _ptr(qweight), _ptr(cherry_weight), _ptr(cherry_indices),
                                      _ptr(scaling_factors), stream.data_ptr(), nbytes, k, n, c, g,
                                      _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "prepack_cherryq")
    return stream


def unprepack_cherryq(w_bits, stream, in_features, out_features, num_cherries, group_size):
    """Inverse of prepack_cherryq: (cherry_indices, cherry_weight, qweight, scales), bit for bit
    the buffers the stream was made from."""
    _check(stream, "stream", torch.uint8, 1)
    dev = stream.device
    k, n, c, g = int(in_features), int(out_features), int(num_cherries), int(group_size)
    kn = k - c
    idx = torch.empty(c, dtype=torch.int16, device=dev)
    cw = torch.empty((c, n), dtype=torch.float16, device=dev)
    qweight = torch.empty((kn // 8 * w_bits, n), dtype=torch.uint8, device=dev)
    scales = torch.empty((-(-kn // g), n), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.cherryq_unprepack_f16(w_bits, stream.data_ptr(), stream.numel(), _ptr(qweight), _ptr(cw), _ptr(idx),
                                        _ptr(scales), k, n, c, g, _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "unprepack_cherryq")
    return idx, cw, qweight, scales


def matvec_prepacked_cherryq(w_bits, vec, stream, out, in_features, num_cherries, accumulate=False):
    """out (B, N) = (or +=) vec (B, K) @ W^T over a stream made by prepack_cherryq, 1 <= B <= 16.
    Result and arithmetic contract are those of vecquant{3,4}matmul_cherryq; no workspace, no
    atomics (from 2 rows a scratch buffer for the compacted activations, kept by this module)."""
    _check(vec, "vec", torch.float16, 2)
    dev = vec.device
    _check(stream, "stream", torch.uint8, 1, dev)
    _check(out, "out", torch.float16, 2, dev)
    batch, k = vec.shape
    if k != int(in_features) or out.shape[0] != batch:
        raise RuntimeError(f"matvec_prepacked_cherryq: vec {tuple(vec.shape)} / out {tuple(out.shape)} do not match")
    if batch == 0:
        return
    with torch.cuda.device(dev):
        hs = _current_stream(dev.index)
        if batch == 1:
            rc = _lib.cherryq_matvec_prepacked_f16(w_bits, vec.data_ptr(), stream.data_ptr(), stream.numel(),
                                                   out.data_ptr(), batch, k, out.shape[1], int(num_cherries),
                                                   1 if accumulate else 0, hs)
        else:
            # 2 to 16 rows: the compacted activations pass through a scratch buffer kept per (device, stream)
            nb = _lib.cherryq_prepacked_scratch_bytes(w_bits, batch, k, out.shape[1], int(num_cherries))
            sc = _scratch(dev, hs, nb)
            rc = _lib.cherryq_matmul_prepacked_f16(w_bits, vec.data_ptr(), stream.data_ptr(), stream.numel(),
                                                   out.data_ptr(), batch, k, out.shape[1], int(num_cherries),
                                                   1 if accumulate else 0, None if sc is None else sc.data_ptr(), nb, hs)
    if rc != 0:
        _fail(rc, "matvec_prepacked_cherryq")


FAKE_QUANT_MAX_IN_FEATURES = 65536
FAKE_QUANT_MAX_GROUPS = 4096


def fake_quant_supported(weight, w_bits, group_size) -> bool:
    """Whether fake_quant_cherryq takes this weight (GPU, fp16 or fp32, 2-D, 2..4 bits, within
    the kernel's channel and group limits)."""
    if not (isinstance(weight, torch.Tensor) and weight.is_cuda and weight.dim() == 2):
        return False
    if weight.dtype not in (torch.float16, torch.float32) or w_bits not in (2, 3, 4):
        return False
    k = weight.shape[1]
    g = int(group_size) if int(group_size) > 0 else k
    return 0 < k <= FAKE_QUANT_MAX_IN_FEATURES and -(-k // g) <= FAKE_QUANT_MAX_GROUPS


def fake_quant_cherryq(w_bits, weight, cherry_indices, group_size, ste=False, out=None):
    """The weight the training-side QuantLinear multiplies with: every non-cherry input channel of
    `weight` (out, in; fp16 or fp32) replaced by its group-wise quantise-dequantise value, bit
    for bit what QuantLinear._adjust_weight computes with torch operations
    (llama/cherry_linear.py:77-99, llama/quantizer.py:148-152 and 165-170), in one pass over the
    matrix.  `ste` selects the straight-through arithmetic form (q - w) + w; the gradient is
    the caller's business.  No counterpart in the reference extension."""
    if not isinstance(weight, torch.Tensor) or weight.dtype not in (torch.float16, torch.float32):
        raise RuntimeError("fake_quant_cherryq: weight must be an fp16 or fp32 tensor")
    _check(weight, "weight", weight.dtype, 2)
    dev = weight.device
    n, k = weight.shape
    if cherry_indices is None:
        idx = torch.empty(0, dtype=torch.int32, device=dev)
    else:
        idx = cherry_indices.to(device=dev, dtype=torch.int32).contiguous()
    if out is None:
        out = torch.empty_like(weight)
    else:
        _check(out, "out", weight.dtype, 2, dev)
        if out.shape != weight.shape:
            raise RuntimeError("fake_quant_cherryq: out must have the weight's shape")
    g = int(group_size) if int(group_size) > 0 else k
    fn = _lib.cherryq_fake_quant_f16 if weight.dtype == torch.float16 else _lib.cherryq_fake_quant_f32
    with torch.cuda.device(dev):
        rc = fn(int(w_bits), weight.data_ptr(), _ptr(idx), out.data_ptr(), k, n, idx.numel(), g, int(bool(ste)),
                _current_stream(dev.index))
    if rc != 0:
        _fail(rc, "fake_quant_cherryq")
    return out
