"""Python face of the HIP kernel library: loads ``libburnlm_hip.so`` through ctypes and wraps
each entry point with checks of device, dtype, shape and contiguity.  Kernels run on torch's
current HIP stream.  There is no fallback: without the library, or off the GPU, calls raise."""
from __future__ import annotations

import ctypes
import threading

import torch

from . import build as _build

ABI_VERSION = 38
_lib = None
_lock = threading.Lock()

_c_int, _c_float, _c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_void_p


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


_SIGNATURES = {
    "blm_embed_gather": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_float, _c_void_p],
    "blm_embed_gather_from": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                              _c_int, _c_float, _c_void_p],
    "blm_input_conv": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p,
                       _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "blm_residual_add": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int,
                         _c_int, _c_void_p],
    "blm_side_gate": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                      _c_int, _c_int, _c_void_p],
    "blm_rms_scale": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
    "blm_clamped_glu": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p],
    "blm_moe_route": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
    "blm_moe_gate": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_gla_scan": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_float, _c_void_p, _c_void_p,
                     _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                     _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_float, _c_int, _c_int, _c_void_p],
    "blm_lightning_chunks_init": [],
    "blm_lightning_chunks_supported": [_c_int, _c_int],
    "blm_lightning_chunks": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                             _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                             _c_int, _c_int, _c_int, _c_void_p],
    "blm_qkv_prepare": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int,
                        _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                        _c_void_p, _c_void_p],
    "blm_sigmoid_gate": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_gelu_glu": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "blm_softcap": [_c_void_p, ctypes.c_longlong, _c_float, _c_void_p],
    "blm_rmsnorm_rows": [_c_void_p, _c_int, _c_int, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_void_p],
    "blm_add_gated_rmsnorm": [_c_void_p, _c_void_p, _c_int, _c_int, ctypes.c_longlong, _c_void_p, _c_void_p, _c_float,
                              _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    "blm_scaled_add": [_c_void_p, _c_int, _c_int, _c_int] + [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int] * 4
                      + [_c_void_p],
    "blm_moe_route_grouped": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int,
                              _c_void_p],
    "blm_sink_attn_mfma_supported": [_c_int, _c_int],
    "blm_sink_attn_mfma": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                           _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                           _c_int, _c_float, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p],
    "blm_sink_attn": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                      _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                      _c_void_p],
    "blm_streams_norm": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, ctypes.c_longlong, _c_void_p, _c_void_p, _c_void_p,
                         _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_float,
                         _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    "blm_token_shift": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p,
                        _c_int, _c_int, _c_void_p],
    "blm_xielu": [_c_void_p, _c_void_p, _c_int, ctypes.c_longlong, _c_float, _c_float, _c_void_p],
    "blm_latent_write": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_float, _c_void_p,
                         _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_latent_attn_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int,
                             _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p, _c_void_p, _c_void_p],
    "blm_latent_attn_mfma_supported": [_c_int, _c_int],
    "blm_head_project": [_c_void_p, _c_int, ctypes.c_longlong, _c_int, _c_void_p, _c_int, _c_void_p, _c_int,
                         ctypes.c_longlong, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_latent_attn": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_int,
                        _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    "blm_hgrn2_scan": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_void_p,
                       _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_conv_prepare": [_c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                         _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_delta_scan": [_c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                       _c_void_p, _c_float, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                       _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_add_rmsnorm": [_c_void_p, _c_void_p, _c_int, _c_int, ctypes.c_longlong, _c_void_p, _c_int, _c_void_p, _c_int,
                        _c_void_p, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    "blm_rope_kv_write": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                          _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "blm_swiglu": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "blm_attn_paged": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int,
                       _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                       _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    "blm_attn_decode": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int,
                        _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    "blm_attn_decode_supported": [_c_int, _c_int, _c_int],
    "blm_attn_prefill_mfma_supported": [_c_int, _c_int, _c_int],
    "blm_attn_prefill_mfma": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int,
                              _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                              _c_int, _c_int, _c_void_p, _c_void_p],
    "blm_gemm_tiled": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                       _c_int, _c_int, _c_void_p],
    "blm_gemv_skinny": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                        _c_int, _c_int, _c_void_p],
    "blm_gemv_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                      _c_int, _c_void_p],
    "blm_gemv_mfma_supported": [_c_int, _c_int, _c_int],
    "blm_gemv_mfma_geometry": [_c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p],
    "blm_gemm_mfma_init": [],
    "blm_gemm_rows_init": [],
    "blm_gemm_rows": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                      _c_int, _c_void_p],
    "blm_attn_paged_init": [],
    "blm_sink_attn_mfma_init": [],
    "blm_gemm_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                      _c_int, _c_int, _c_int, _c_void_p],
    "blm_gemv_mfma_group_limit": [_c_int],
    "blm_gemv_qkv_rope_supported": [_c_int, _c_int, _c_int, _c_int],
    "blm_gemv_qkv_rope": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                          _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_int, _c_void_p],
    "blm_gemm_rows_qkv_rope": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                               _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                               _c_int, _c_int, _c_int, _c_void_p],
    "blm_argmax": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p],
    "blm_probe_read": [_c_void_p, ctypes.c_longlong, _c_void_p, _c_int, _c_void_p],
    "blm_probe_mfma": [_c_int, _c_int, _c_int, _c_void_p, _c_void_p],
    "blm_static_scratch_init": [],
    "blm_argmax_static": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "blm_sample": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void_p, _c_void_p,
                   _c_void_p],
}


def library():
    """The loaded kernel library; built from source at the first call if it is not there."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_built()
                lib = ctypes.CDLL(path)
                lib.blm_last_error.restype = ctypes.c_char_p
                lib.blm_abi_version.restype = _c_int
                if lib.blm_abi_version() != ABI_VERSION:
                    raise KernelError(f"{path} has ABI {lib.blm_abi_version()}, expected {ABI_VERSION}: rebuild it")
                for name, sig in _SIGNATURES.items():
                    fn = getattr(lib, name)
                    fn.argtypes = sig
                    fn.restype = _c_int
                lib.blm_sample_scratch_bytes.argtypes = [_c_int, _c_int]
                lib.blm_sample_scratch_bytes.restype = ctypes.c_longlong
                lib.blm_attn_prefill_blocks32.argtypes = [_c_int] * 5
                lib.blm_attn_prefill_blocks32.restype = ctypes.c_longlong
                _lib = lib
    return _lib


def library_file():
    return _build.lib_path()


DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def _code(t):
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not supported by the kernels (float32 or bfloat16)") from None


def _gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("the kernels run on the GPU only: got a tensor on " + str(t.device))


def _contig(name, t):
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


def _i32(name, t, n=None):
    if t.dtype != torch.int32:
        raise KernelError(f"{name} must be int32, got {t.dtype}")
    _contig(name, t)
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} elements, needs {n}")


def _stream():
    """The current HIP stream's handle.  torch's raw accessor costs a fraction of a microsecond; the
    Stream object of torch.cuda.current_stream() several, at every launch."""
    return _raw_stream(torch.cuda.current_device())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda i: torch.cuda.current_stream(i).cuda_stream)


def _call(name, *args):
    lib = library()
    if len(args) != len(_SIGNATURES[name]):
        # ctypes would pass the surplus as 32-bit integers and cut pointers (a stream handle) short
        raise KernelError(f"{name}: {len(args)} arguments given, its signature has {len(_SIGNATURES[name])}")
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.blm_last_error().decode())


def _ptr(t):
    return 0 if t is None else t.data_ptr()


ARRIVAL_COUNTERS = 1 << 16
_arrivals = {}


def arrival_counters(device):
    """Zeroed int32 counters of a device, for kernels whose blocks count themselves in so that the
    last one finishes a shared result.  Every such kernel leaves them zero again, so all of them
    share one buffer; launches that use it must not overlap in time (one stream at a time).  It is
    allocated at the first call, which must not be under graph capture (Runtime() makes that call)."""
    device = torch.device(device)
    key = device.index if device.index is not None else torch.cuda.current_device()
    buf = _arrivals.get(key)
    if buf is None:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("arrival_counters: the first call for a device must come before any graph capture")
        buf = _arrivals[key] = torch.zeros(ARRIVAL_COUNTERS, dtype=torch.int32, device=torch.device("cuda", key))
    return buf


def _check_planes(who, kcache, vcache, nkv, page_size, hd):
    """Key plane [pages, kv_heads, page, head_dim]; value plane [pages, kv_heads, head_dim, page]."""
    if tuple(kcache.shape[1:]) != (nkv, page_size, hd) or tuple(vcache.shape) != (kcache.shape[0], nkv, hd, page_size):
        raise KernelError(f"{who}: cache planes {tuple(kcache.shape)} / {tuple(vcache.shape)} do not fit keys "
                          f"[pages, {nkv}, {page_size}, {hd}] and values [pages, {nkv}, {hd}, {page_size}]")


# ------------------------------------------------------------------------------------------
def _embed_shape(who, table, out_h):
    """(T, D, copies) of an embedding output [T, D] or [T, copies, D]."""
    if out_h.dtype != torch.float32 or out_h.dim() not in (2, 3) or table.shape[1] != out_h.shape[-1]:
        raise KernelError(f"{who}: h must be float32 [T, D] or [T, copies, D] with D the table's width")
    return out_h.shape[0], out_h.shape[-1], (out_h.shape[1] if out_h.dim() == 3 else 1)


def embed_gather(table, ids, out_h, scale=1.0):
    """out_h[t, :] = table[ids[t], :] * scale as float32 (out_h [T, copies, D]: every copy alike).  ids must already
    be checked against the vocabulary."""
    _gpu(table, ids, out_h)
    T, D, copies = _embed_shape("embed_gather", table, out_h)
    _i32("ids", ids, T)
    _contig("table", table); _contig("h", out_h)
    _call("blm_embed_gather", table.data_ptr(), _code(table), ids.data_ptr(), out_h.data_ptr(), T, D, copies, float(scale),
          _stream())
    return out_h


def embed_gather_from(table, ids, source_rows, source_cell, out_h, scale=1.0):
    """Like embed_gather, but row t's token is taken on the device where source_rows[t] >= 0: it is
    element source_rows[t] of the int32 array whose address stands in source_cell (an int64 tensor of
    one element on the device).  A token outside the vocabulary gives a row of NaN."""
    _gpu(table, ids, source_rows, source_cell, out_h)
    T, D, copies = _embed_shape("embed_gather_from", table, out_h)
    _i32("ids", ids, T)
    _i32("source_rows", source_rows, T)
    _contig("table", table); _contig("h", out_h)
    if source_cell.dtype != torch.int64 or source_cell.numel() != 1:
        raise KernelError("embed_gather_from: the cell is one int64 on the device")
    _call("blm_embed_gather_from", table.data_ptr(), _code(table), ids.data_ptr(), source_rows.data_ptr(),
          source_cell.data_ptr(), out_h.data_ptr(), T, D, table.shape[0], copies, float(scale), _stream())
    return out_h


def add_rmsnorm(h, delta, gamma, eps, out, rows=None, write_h=True, gate=None, gate_bias=None, mult=1.0):
    """v = h[r] (+ delta[r]); h[r] = v if write_h; out[i] = v / sqrt(mean(v^2) + eps) * gamma,
    with r = rows[i] if rows is given, else i.  h is the float32 residual stream.  delta: [T, D] in
    out's dtype, or float32 [planes, T, D] whose planes are summed (partial matrix products).
    gate ([T, D] in out's dtype; with gate_bias float32 [D] or None): the summed delta joins as
    mult * delta * sigmoid(gate + gate_bias)."""
    _gpu(h, delta, gamma, out, rows, gate, gate_bias)
    D = h.shape[1]
    n_out = out.shape[0]
    if h.dtype != torch.float32:
        raise KernelError("add_rmsnorm: the residual stream must be float32")
    _contig("h", h); _contig("out", out); _contig("gamma", gamma)
    if gamma.numel() != D or out.shape[1] != D:
        raise KernelError(f"add_rmsnorm: width mismatch h={D} gamma={gamma.numel()} out={out.shape[1]}")
    planes, stride, dcode = 1, 0, 0
    if delta is not None:
        _contig("delta", delta)
        if delta.dim() == 3:
            if delta.shape[1:] != h.shape or delta.dtype != torch.float32:
                raise KernelError("add_rmsnorm: partial deltas must be float32 [planes, T, D]")
            planes, stride = delta.shape[0], h.shape[0] * D
        elif delta.shape != h.shape or delta.dtype not in (out.dtype, torch.float32):
            raise KernelError("add_rmsnorm: delta must match h in shape and be of out's dtype or float32")
        dcode = _code(delta)
    if rows is not None:
        _i32("rows", rows, n_out)
    elif n_out != h.shape[0]:
        raise KernelError("add_rmsnorm: out needs one row per row of h when rows is not given")
    if gate is not None:
        _contig("gate", gate)
        if delta is None or gate.shape != h.shape or gate.dtype != out.dtype:
            raise KernelError("add_rmsnorm: a gate comes with a delta, is [T, D] and of out's dtype")
        if gate_bias is not None:
            _f32("gate_bias", gate_bias, D)
        _call("blm_add_gated_rmsnorm", h.data_ptr(), _ptr(delta), dcode, planes, stride, gate.data_ptr(), _ptr(gate_bias),
              float(mult), gamma.data_ptr(), _code(gamma), out.data_ptr(), _code(out), _ptr(rows), n_out, D, float(eps),
              1 if write_h else 0, _stream())
        return out
    _call("blm_add_rmsnorm", h.data_ptr(), _ptr(delta), dcode, planes, stride, gamma.data_ptr(), _code(gamma),
          out.data_ptr(), _code(out), _ptr(rows), n_out, D, float(eps), 1 if write_h else 0, _stream())
    return out


def rope_kv_write(qkv, positions, token_seq, block_table, cos_sin, kcache, vcache, page_size,
                  nh, nkv, hd, pairing, write_kv=True):
    """Rotate q (in place) and k of each token by its position's angles and store k, v in the
    paged cache.  cos_sin: float32 [positions, hd/2, 2].  Key plane [pages, nkv, page, hd]; value
    plane [pages, nkv, hd, page]."""
    _gpu(qkv, positions, token_seq, block_table, cos_sin, kcache, vcache)
    T = qkv.shape[0]
    _contig("qkv", qkv); _contig("cos_sin", cos_sin); _contig("kcache", kcache); _contig("vcache", vcache)
    if qkv.shape[1] != (nh + 2 * nkv) * hd:
        raise KernelError(f"rope_kv_write: qkv row is {qkv.shape[1]}, expected {(nh + 2 * nkv) * hd}")
    _i32("positions", positions, T); _i32("token_seq", token_seq, T); _i32("block_table", block_table)
    if cos_sin.dtype != torch.float32 or cos_sin.shape[1:] != (hd // 2, 2):
        raise KernelError("rope_kv_write: cos_sin must be float32 [positions, head_dim/2, 2]")
    if kcache.dtype != qkv.dtype or vcache.dtype != qkv.dtype:
        raise KernelError("rope_kv_write: cache and activations must share a dtype")
    _check_planes("rope_kv_write", kcache, vcache, nkv, page_size, hd)
    _call("blm_rope_kv_write", qkv.data_ptr(), _code(qkv), positions.data_ptr(), token_seq.data_ptr(),
          block_table.data_ptr(), block_table.shape[1], cos_sin.data_ptr(), kcache.data_ptr(), vcache.data_ptr(),
          page_size, T, nh, nkv, hd, pairing, 1 if write_kv else 0, _stream())


def swiglu(gate_up, out):
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _gpu(gate_up, out)
    T, I = out.shape
    _contig("gate_up", gate_up); _contig("out", out)
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError("swiglu: gate_up must be [T, 2I] of out's dtype")
    _call("blm_swiglu", gate_up.data_ptr(), out.data_ptr(), _code(out), T, I, _stream())
    return out


def attn_paged(q, q_row_stride, out, positions, token_seq, block_table, kcache, vcache, page_size,
               nh, nkv, hd, scale, window=0, n_splits=1):
    """Attention of every query token over its sequence's cached keys (generic kernel).
    q: first nh*hd columns of rows with stride q_row_stride; out: [T, nh*hd].  n_splits > 1 cuts
    every key range into that many pieces for different wavefronts (few tokens over long ranges)."""
    _gpu(q, out, positions, token_seq, block_table, kcache, vcache)
    T = out.shape[0]
    _contig("out", out); _contig("kcache", kcache); _contig("vcache", vcache)
    if out.shape[1] != nh * hd or out.dtype != q.dtype or kcache.dtype != q.dtype:
        raise KernelError("attn_paged: out must be [T, heads*head_dim] and share q's dtype with the cache")
    if q.stride(-1) != 1 or q_row_stride < nh * hd:
        raise KernelError("attn_paged: q rows must be contiguous and at least heads*head_dim long")
    _check_planes("attn_paged", kcache, vcache, nkv, page_size, hd)
    _i32("positions", positions, T); _i32("token_seq", token_seq, T); _i32("block_table", block_table)
    n_splits = max(1, int(n_splits))
    part_o = part_ml = arrivals = None
    if n_splits > 1:
        arrivals = arrival_counters(out.device)
        if T * nh > arrivals.numel():
            n_splits = 1      # more (token, head) pairs than counters: enough parallel work without cutting
        else:
            part_o = torch.empty(T * nh * n_splits * hd, dtype=torch.float32, device=out.device)
            part_ml = torch.empty(T * nh * n_splits * 2, dtype=torch.float32, device=out.device)
    _call("blm_attn_paged", q.data_ptr(), q_row_stride, out.data_ptr(), _code(out), positions.data_ptr(),
          token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], kcache.data_ptr(), vcache.data_ptr(),
          page_size, T, nh, nkv, hd, float(scale), int(window), n_splits, _ptr(part_o), _ptr(part_ml),
          _ptr(arrivals if n_splits > 1 else None), _stream())
    return out


def attn_decode_supported(dtype, hd, page_size=64):
    """Whether the matrix-core decode kernel takes this case (else the generic kernel does)."""
    return dtype in DTYPE_CODE and bool(library().blm_attn_decode_supported(DTYPE_CODE[dtype], int(hd), int(page_size)))


def attn_prefill_mfma_supported(dtype, hd, page_size=64):
    return dtype in DTYPE_CODE and bool(
        library().blm_attn_prefill_mfma_supported(DTYPE_CODE[dtype], int(hd), int(page_size)))


def attn_prefill_queries(n_seqs, max_new, nh, nkv, hd, compute_units):
    """Query rows per wavefront that attn_prefill_mfma should take for a step.  With 32 every key and value
    fragment taken from shared memory serves twice the queries, which is worth 5-12 % where the step is bound
    by the work (several rounds of blocks); with 16 a page takes a wavefront less long, which is worth 15-25 %
    where all blocks run at once and the step lasts as long as its longest query tile.  So: 32 once that
    form's blocks are 8 times the compute units (4 times for heads above 64, whose blocks are two to a
    compute unit), or 2 times with a prompt of 3,072 tokens and more."""
    blocks32 = library().blm_attn_prefill_blocks32(int(n_seqs), int(max_new), int(nh), int(nkv), int(hd))
    rounds = 8 if hd <= 64 else 4
    units = int(compute_units)
    return 32 if blocks32 >= rounds * units or (max_new >= 3072 and blocks32 >= 2 * units) else 16


def attn_prefill_mfma(q, q_row_stride, out, positions, cu_seqlens, block_table, kcache, vcache, page_size,
                      n_seqs, max_new, nh, nkv, hd, scale, window=0, queries=16, sinks=None):
    """Causal attention of packed sequences over their cached keys on the matrix cores (bfloat16).
    Rows cu_seqlens[b] .. cu_seqlens[b+1] of q and out belong to sequence b; max_new is the most
    rows any sequence has.  queries: 16 or 32 query rows per wavefront (attn_prefill_queries chooses).
    sinks (float32 [heads]): the softmax's denominator also holds exp(sinks[h]), a logit without key or value."""
    _gpu(q, out, positions, cu_seqlens, block_table, kcache, vcache, sinks)
    if sinks is not None:
        _f32("sinks", sinks, nh)
    T = out.shape[0]
    _contig("out", out); _contig("kcache", kcache); _contig("vcache", vcache)
    if out.shape[1] != nh * hd or out.dtype != q.dtype or kcache.dtype != q.dtype:
        raise KernelError("attn_prefill_mfma: out must be [T, heads*head_dim] and share q's dtype with the cache")
    if q.stride(-1) != 1 or q_row_stride < nh * hd:
        raise KernelError("attn_prefill_mfma: q rows must be contiguous and at least heads*head_dim long")
    _check_planes("attn_prefill_mfma", kcache, vcache, nkv, page_size, hd)
    _i32("positions", positions, T); _i32("cu_seqlens", cu_seqlens, n_seqs + 1); _i32("block_table", block_table)
    if block_table.shape[0] < n_seqs:
        raise KernelError("attn_prefill_mfma: the page table has fewer rows than there are sequences")
    _call("blm_attn_prefill_mfma", q.data_ptr(), q_row_stride, out.data_ptr(), _code(out), positions.data_ptr(),
          cu_seqlens.data_ptr(), block_table.data_ptr(), block_table.shape[1], kcache.data_ptr(), vcache.data_ptr(),
          page_size, int(n_seqs), int(max_new), nh, nkv, hd, float(scale), int(window), int(queries), _ptr(sinks), _stream())
    return out


def attn_decode(q, q_row_stride, out, positions, token_seq, block_table, kcache, vcache, page_size,
                nh, nkv, hd, scale, window=0, n_splits=1, sinks=None):
    """Attention for few query tokens over long key ranges, the key range cut into n_splits.  sinks: as for
    attn_prefill_mfma."""
    _gpu(q, out, positions, token_seq, block_table, kcache, vcache, sinks)
    if sinks is not None:
        _f32("sinks", sinks, nh)
    T = out.shape[0]
    _contig("out", out); _contig("kcache", kcache); _contig("vcache", vcache)
    if out.shape[1] != nh * hd or out.dtype != q.dtype or kcache.dtype != q.dtype:
        raise KernelError("attn_decode: out must be [T, heads*head_dim] and share q's dtype with the cache")
    if q.stride(-1) != 1 or q_row_stride < nh * hd:
        raise KernelError("attn_decode: q rows must be contiguous and at least heads*head_dim long")
    _check_planes("attn_decode", kcache, vcache, nkv, page_size, hd)
    _i32("positions", positions, T); _i32("token_seq", token_seq, T); _i32("block_table", block_table)
    n_splits = decode_pieces(T, nh, nkv, n_splits, arrival_counters(out.device).numel())
    part_o = part_ml = arrivals = None
    if n_splits > 1:    # an uncut key range leaves no partial result and counts nobody in
        part_o = torch.empty(T * nh * n_splits * hd, dtype=torch.float32, device=out.device)
        part_ml = torch.empty(T * nh * n_splits * 2, dtype=torch.float32, device=out.device)
        arrivals = arrival_counters(out.device)
    _call("blm_attn_decode", q.data_ptr(), q_row_stride, out.data_ptr(), _code(out), positions.data_ptr(),
          token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], kcache.data_ptr(), vcache.data_ptr(),
          page_size, T, nh, nkv, hd, float(scale), int(window), n_splits, _ptr(part_o), _ptr(part_ml),
          _ptr(arrivals), _ptr(sinks), _stream())
    return out


def decode_pieces(T, nh, nkv, n_splits, n_counters):
    """Into how many pieces attn_decode really cuts the key ranges: as asked, but not at all when
    the (token, head tile) pairs outnumber the arrival counters (so many pairs are work enough for
    the whole chip without cutting, as attn_paged decides too)."""
    n_splits = max(1, int(n_splits))
    if n_splits > 1 and T * nkv * ((nh // nkv + 15) // 16) > n_counters:
        return 1
    return n_splits


def _check_mm(a, w, out):
    _gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelError(f"matrix product: shapes a={tuple(a.shape)} w={tuple(w.shape)} out={tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("matrix product: a and out need unit stride along their rows")
    _contig("w", w)
    return M, N, K


def gemm_tiled(a, w, out):
    """out[M,N] = a[M,K] @ w[N,K]^T with float accumulation by plain fused multiply-adds."""
    M, N, K = _check_mm(a, w, out)
    _call("blm_gemm_tiled", a.data_ptr(), _code(a), w.data_ptr(), _code(w), out.data_ptr(), _code(out),
          M, N, K, a.stride(0), out.stride(0), _stream())
    return out


def gemv_skinny(a, w, out):
    """The same product for M <= 8 rows; streams w once."""
    M, N, K = _check_mm(a, w, out)
    _call("blm_gemv_skinny", a.data_ptr(), _code(a), w.data_ptr(), _code(w), out.data_ptr(), _code(out),
          M, N, K, a.stride(0), out.stride(0), _stream())
    return out


def gemv_mfma_supported(M, N, K):
    """Whether gemv_mfma takes M rows with all of K in one group."""
    return bool(library().blm_gemv_mfma_supported(int(M), int(N), int(K)))


def gemv_mfma_group_limit(M):
    """The largest K that one K-group of gemv_mfma may span for M rows (0: M out of range)."""
    return int(library().blm_gemv_mfma_group_limit(int(M)))


def gemv_mfma_geometry(M, N, K, groups=1):
    """(blocks over all groups, wavefronts per block) that gemv_mfma launches for M rows of a [N, K]
    matrix in that many groups of K, or None if a group's stretch of K is beyond what it takes."""
    blocks, waves = ctypes.c_int(0), ctypes.c_int(0)
    ok = library().blm_gemv_mfma_geometry(int(M), int(N), int(K), int(groups), ctypes.byref(blocks), ctypes.byref(waves))
    return (blocks.value, waves.value) if ok else None


def pack_weight(w, gated=False):
    """Copy of a bfloat16 weight matrix [N, K] in the order the matrix-core skinny product streams
    it: packed[tile, step, lane, e] = w[tile*16 + lane%16, step*32 + (lane//16)*8 + e], with N
    padded to a multiple of 16 and K to a multiple of 32 by zeros.  Returns a flat tensor.
    gated=True: w is [gate rows; up rows]; its rows are first re-ordered into blocks of 8 gate rows
    followed by the 8 matching up rows, so that each tile holds 8 gated pairs (gemv_mfma gated=True)."""
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise KernelError("pack_weight: needs a bfloat16 matrix")
    N, K = w.shape
    if gated:
        if N % 16:
            raise KernelError("pack_weight: a gated matrix needs a multiple of 8 features")
        half = N // 2
        w = torch.stack([w[:half].view(half // 8, 8, K), w[half:].view(half // 8, 8, K)], dim=1).reshape(N, K)
    Np, Kp = (N + 15) // 16 * 16, (K + 31) // 32 * 32
    if (Np, Kp) != (N, K):
        padded = torch.zeros(Np, Kp, dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    # [tile, row, step, kg, e] -> [tile, step, kg, row, e]
    return w.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1)


def gemv_mfma(a, packed, out, K, gated=False, activation="silu"):
    """bfloat16 product for M <= 64 rows on the matrix cores; streams the packed weights once (17 to 64
    rows: K at most 2048 per group, see gemv_mfma_group_limit).
    packed: pack_weight(w) of w [N, K].  out: bfloat16 or float32 [M, N], or float32
    [groups, M, N]: K is then cut into that many groups whose partial products fill the planes of
    out (the reader sums them).  gated=True: packed = pack_weight(w, gated=True) of a [2I, K] matrix
    and out is [M, I] = act(a gate^T) * (a up^T) with act = silu, or (activation="gelu_tanh") the tanh form of GELU."""
    _gpu(a, packed, out)
    if activation not in ("silu", "gelu_tanh"):
        raise KernelError(f"gemv_mfma: activation {activation!r} unknown (silu, gelu_tanh)")
    groups = 1
    if out.dim() == 3:
        groups = out.shape[0]
        if out.dtype != torch.float32 or not out.is_contiguous():
            raise KernelError("gemv_mfma: partial outputs must be contiguous float32 [groups, M, N]")
    M = out.shape[-2]
    N = out.shape[-1] * (2 if gated else 1)
    if a.shape != (M, K):
        raise KernelError(f"gemv_mfma: shapes a={tuple(a.shape)} out={tuple(out.shape)} K={K} do not fit")
    if packed.numel() != ((N + 15) // 16) * ((K + 31) // 32) * 512 or not packed.is_contiguous():
        raise KernelError(f"gemv_mfma: the packed weights have {packed.numel()} elements, not those of a "
                          f"[{N}, {K}] matrix")
    if a.stride(1) != 1 or out.stride(-1) != 1:
        raise KernelError("gemv_mfma: a and out need unit stride along their rows")
    if a.dtype != torch.bfloat16 or packed.dtype != torch.bfloat16:
        raise KernelError("gemv_mfma: operands must be bfloat16")
    _call("blm_gemv_mfma", a.data_ptr(), packed.data_ptr(), out.data_ptr(), _code(out), M, N, K, a.stride(0),
          out.stride(-2), (2 if activation == "gelu_tanh" else 1) if gated else 0, groups, _stream())
    return out


GEMM_TILES = {(128, 128): 0, (256, 128): 1, (256, 256): 2, (128, 128, 4): 3, (128, 64, 6): 4}
_gemm_ready = set()


def gemm_mfma_init(device=None):
    """Once per device, outside any stream capture, before the first gemm_mfma: its kernels use more
    shared memory than a kernel gets without asking."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _gemm_ready:
        with torch.cuda.device(index):
            _call("blm_gemm_mfma_init")
        _gemm_ready.add(index)


_attn_ready = set()


def attn_paged_init(device=None):
    """Once per device, outside any stream capture: lets attn_paged stage the values of head sizes
    above 62 (up to 139) through shared memory."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _attn_ready:
        with torch.cuda.device(index):
            _call("blm_attn_paged_init")
        _attn_ready.add(index)


_static_ready = set()


def static_scratch_init(device=None):
    """Once per device, outside any stream capture: the library looks up where its own scratch array
    lies on that device (blm_argmax_static, the entry point for callers that cannot allocate)."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _static_ready:
        with torch.cuda.device(index):
            _call("blm_static_scratch_init")
        _static_ready.add(index)


def gemm_mfma(a, w, out, gated=False, tile=(128, 128), activation="silu"):
    """bfloat16 product for many rows on the matrix cores: out = a[M, K] @ w[N, K]^T, with w as the
    checkpoint stores it.  out: bfloat16 or float32 [M, N], or float32 [groups, M, N] partial
    products over that many groups of K (the reader sums them).  gated=True: w is [gate rows; up
    rows] ([2I, K]) and out is [M, I] = act(a gate^T) * (a up^T), act = silu or (activation="gelu_tanh") the tanh form
    of GELU.  tile: rows x columns of out (of
    gate and up columns together when gated) per block, one of GEMM_TILES; a third number is the depth of
    the ring of K stages (deep rings for products of few tiles, which wait for memory, not for the matrix cores)."""
    _gpu(a, w, out)
    gemm_mfma_init(a.device)
    groups = 1
    if out.dim() == 3:
        groups = out.shape[0]
        if out.dtype != torch.float32 or not out.is_contiguous():
            raise KernelError("gemm_mfma: partial outputs must be contiguous float32 [groups, M, N]")
    M, N = out.shape[-2], out.shape[-1]
    K = a.shape[1]
    if a.shape[0] != M or w.dim() != 2 or w.shape != (N * (2 if gated else 1), K):
        raise KernelError(f"gemm_mfma: shapes a={tuple(a.shape)} w={tuple(w.shape)} out={tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(-1) != 1:
        raise KernelError("gemm_mfma: a, w and out need unit stride along their rows")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_mfma: operands must be bfloat16")
    if tile not in GEMM_TILES:
        raise KernelError(f"gemm_mfma: tile {tile} is not one of {sorted(GEMM_TILES)}")
    _call("blm_gemm_mfma", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out), M, N, K, a.stride(0), w.stride(0),
          out.stride(-2), (2 if activation == "gelu_tanh" else 1) if gated else 0, groups, GEMM_TILES[tile], _stream())
    return out


_rows_ready = set()


def gemm_rows_init(device=None):
    """Once per device, outside any stream capture, before the first gemm_rows (its rings of stages
    take more shared memory than a kernel gets without asking)."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _rows_ready:
        with torch.cuda.device(index):
            _call("blm_gemm_rows_init")
        _rows_ready.add(index)


def gemm_rows(a, w, out, gated=False, columns=64):
    """bfloat16 product for few rows (made for 17 to 64; up to 256 as one block for every 64 rows) whose loads
    never stop for a barrier: out = a[M, K] @ w[N, K]^T, w as the checkpoint stores it.  out: bfloat16 or float32 [M, N], or float32 [groups, M, N] partial
    products over that many groups of K (the reader sums them).  gated=True: w is [gate rows; up rows]
    ([2I, K]) and out is [M, I] = silu(a gate^T) * (a up^T).  columns: 64 or (without gating) 32 columns
    of out (of gate and up together when gated) per block."""
    _gpu(a, w, out)
    gemm_rows_init(a.device)
    groups = 1
    if out.dim() == 3:
        groups = out.shape[0]
        if out.dtype != torch.float32 or not out.is_contiguous():
            raise KernelError("gemm_rows: partial outputs must be contiguous float32 [groups, M, N]")
    M, N = out.shape[-2], out.shape[-1]
    K = a.shape[1]
    if a.shape[0] != M or w.dim() != 2 or w.shape != (N * (2 if gated else 1), K):
        raise KernelError(f"gemm_rows: shapes a={tuple(a.shape)} w={tuple(w.shape)} out={tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(-1) != 1:
        raise KernelError("gemm_rows: a, w and out need unit stride along their rows")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_rows: operands must be bfloat16")
    _call("blm_gemm_rows", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out), M, N, K, a.stride(0), w.stride(0),
          out.stride(-2), 1 if gated else 0, groups, int(columns), _stream())
    return out


def gemv_qkv_rope_supported(M, K, hd, pairing):
    """Up to 16 rows: pairing 0 (adjacent lanes) with head_dim a multiple of 16, pairing 1 (half a head
    apart) with a multiple of 32, K up to 4096.  17 to 64 rows: pairing 0; K up to 4096 for at most 32
    rows, up to 2048 beyond."""
    return bool(library().blm_gemv_qkv_rope_supported(int(M), int(K), int(hd), int(pairing)))


def gemv_qkv_rope(x, packed, qkv_out, positions, token_seq, block_table, cos_sin, kcache, vcache, page_size,
                  nh, nkv, hd, pairing, write_kv=True):
    """Decode: x [M<=64, K] @ W_qkv^T on the matrix cores, rotary encoding of q and k on the float
    results, q into qkv_out[:, :nh*hd], k and v into their cache pages, all in one kernel.
    packed: pack_weight of W_qkv [(nh + 2 nkv) * hd, K]."""
    _gpu(x, packed, qkv_out, positions, token_seq, block_table, cos_sin, kcache, vcache)
    M, K = x.shape
    N = (nh + 2 * nkv) * hd
    if x.dtype != torch.bfloat16 or packed.dtype != torch.bfloat16 or qkv_out.dtype != torch.bfloat16:
        raise KernelError("gemv_qkv_rope: operands must be bfloat16")
    if packed.numel() != (N // 16) * ((K + 31) // 32) * 512 or not packed.is_contiguous():
        raise KernelError(f"gemv_qkv_rope: the packed weights are not those of a [{N}, {K}] matrix")
    if qkv_out.shape[0] != M or qkv_out.stride(1) != 1 or qkv_out.shape[1] < nh * hd or x.stride(1) != 1:
        raise KernelError("gemv_qkv_rope: qkv_out must be [M, >= heads*head_dim] with unit stride along rows")
    _i32("positions", positions, M); _i32("token_seq", token_seq, M); _i32("block_table", block_table)
    if cos_sin.dtype != torch.float32 or cos_sin.shape[1:] != (hd // 2, 2) or not cos_sin.is_contiguous():
        raise KernelError("gemv_qkv_rope: cos_sin must be contiguous float32 [positions, head_dim/2, 2]")
    if kcache.dtype != torch.bfloat16:
        raise KernelError("gemv_qkv_rope: the cache must be bfloat16")
    _contig("kcache", kcache); _contig("vcache", vcache)
    _check_planes("gemv_qkv_rope", kcache, vcache, nkv, page_size, hd)
    _call("blm_gemv_qkv_rope", x.data_ptr(), packed.data_ptr(), qkv_out.data_ptr(), positions.data_ptr(),
          token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], cos_sin.data_ptr(), kcache.data_ptr(),
          vcache.data_ptr(), page_size, M, K, x.stride(0), qkv_out.stride(0), nh, nkv, hd, pairing,
          1 if write_kv else 0, _stream())
    return qkv_out


def gemm_rows_qkv_rope(x, w, qkv_out, positions, token_seq, block_table, cos_sin, kcache, vcache, page_size,
                       nh, nkv, hd, write_kv=True, columns=32, rows=64):
    """17 to 256 rows: x [M, K] @ W_qkv^T (w [(nh + 2 nkv) * hd, K] as bound, rotary partners in adjacent
    rows), rotary encoding of q and k on the float results, q into qkv_out[:, :nh*hd], k and v into
    their cache pages, in one kernel (the product of gemm_rows).  columns: 32 or 64 per block; rows: 64
    staged per block, or 32 (with 32 columns), which is what runs up to 32 rows in any case."""
    _gpu(x, w, qkv_out, positions, token_seq, block_table, cos_sin, kcache, vcache)
    gemm_rows_init(x.device)
    M, K = x.shape
    N = (nh + 2 * nkv) * hd
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or qkv_out.dtype != torch.bfloat16:
        raise KernelError("gemm_rows_qkv_rope: operands must be bfloat16")
    if w.dim() != 2 or w.shape != (N, K) or w.stride(1) != 1:
        raise KernelError(f"gemm_rows_qkv_rope: the weights must be [{N}, {K}] with unit stride along rows, got {tuple(w.shape)}")
    if qkv_out.shape[0] != M or qkv_out.stride(1) != 1 or qkv_out.shape[1] < nh * hd or x.stride(1) != 1:
        raise KernelError("gemm_rows_qkv_rope: qkv_out must be [M, >= heads*head_dim] with unit stride along rows")
    _i32("positions", positions, M); _i32("token_seq", token_seq, M); _i32("block_table", block_table)
    if cos_sin.dtype != torch.float32 or cos_sin.shape[1:] != (hd // 2, 2) or not cos_sin.is_contiguous():
        raise KernelError("gemm_rows_qkv_rope: cos_sin must be contiguous float32 [positions, head_dim/2, 2]")
    if kcache.dtype != torch.bfloat16:
        raise KernelError("gemm_rows_qkv_rope: the cache must be bfloat16")
    _contig("kcache", kcache); _contig("vcache", vcache)
    _check_planes("gemm_rows_qkv_rope", kcache, vcache, nkv, page_size, hd)
    _call("blm_gemm_rows_qkv_rope", x.data_ptr(), w.data_ptr(), qkv_out.data_ptr(), positions.data_ptr(),
          token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], cos_sin.data_ptr(), kcache.data_ptr(),
          vcache.data_ptr(), page_size, M, K, x.stride(0), w.stride(0), qkv_out.stride(0), nh, nkv, hd,
          1 if write_kv else 0, columns, rows, _stream())
    return qkv_out


def argmax(logits, out=None):
    """First index of each row's maximum of float32 logits [R, V] -> int32 [R]."""
    _gpu(logits, out)
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 with unit stride along the vocabulary")
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _i32("out", out, R)
    slice_val = torch.empty(R * 32, dtype=torch.float32, device=logits.device)
    slice_idx = torch.empty(R * 32, dtype=torch.int32, device=logits.device)
    _call("blm_argmax", logits.data_ptr(), out.data_ptr(), R, V, logits.stride(0), slice_val.data_ptr(),
          slice_idx.data_ptr(), _stream())
    return out


def sample(logits, uniforms, temperature, top_p=1.0, out=None):
    """Pick from softmax(logits / temperature) cut to the top-p nucleus at the given uniforms (on the
    GPU, or in pinned host memory, which the kernel reads in place)."""
    _gpu(logits, out)
    if not (uniforms.is_cuda or uniforms.is_pinned()):
        raise KernelError("sample: uniforms must be on the GPU or in pinned host memory")
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 with unit stride along the vocabulary")
    if uniforms.dtype != torch.float32 or uniforms.numel() < R or not uniforms.is_contiguous():
        raise KernelError("sample: uniforms must be contiguous float32 with one value per row")
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _i32("out", out, R)
    counters = arrival_counters(logits.device)
    if R > counters.numel():
        raise KernelError(f"sample: {R} rows are more than the {counters.numel()} counters")
    lib = library()
    scratch = torch.empty((int(lib.blm_sample_scratch_bytes(R, V)) + 7) // 8, dtype=torch.int64, device=logits.device)
    _call("blm_sample", logits.data_ptr(), uniforms.data_ptr(), out.data_ptr(), R, V, logits.stride(0),
          float(temperature), float(top_p), scratch.data_ptr(), counters.data_ptr(), _stream())
    return out


def probe_read(buffer, blocks=2048):
    """Launches the read-only measuring kernel over the whole buffer (see probe.hip); returns the bytes it reads."""
    _gpu(buffer)
    _contig("buffer", buffer)
    n = buffer.numel() * buffer.element_size() // 16 * 16
    sink = _probe_sink(buffer.device)
    _call("blm_probe_read", buffer.data_ptr(), n, sink.data_ptr(), int(blocks), _stream())
    return n


def probe_mfma(iters=4096, blocks=2048, device="cuda", random_operands=False):
    """Launches the matrix-instruction measuring kernel (on the same small operands every time, or on
    random ones that change with every instruction); returns the floating-point operations it does."""
    sink = _probe_sink(torch.device(device))
    _call("blm_probe_mfma", int(iters), int(blocks), 1 if random_operands else 0, sink.data_ptr(), _stream())
    return blocks * 4 * iters * 4 * 2 * 32 * 32 * 16


_sinks = {}


def _probe_sink(device):
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _sinks:
        _sinks[index] = torch.zeros(4, dtype=torch.float32, device=f"cuda:{index}")
    return _sinks[index]


# ------------------------------------------------------------------------------------------
# residual arrangements with several streams, token shift, xIELU
def _f32(name, t, n=None):
    if t.dtype != torch.float32:
        raise KernelError(f"{name} must be float32, got {t.dtype}")
    _contig(name, t)
    if n is not None and t.numel() != n:
        raise KernelError(f"{name} has {t.numel()} elements, needs {n}")


def streams_norm(x, out, gamma, beta, eps, read=None, pending=None, rows=None, write_x=True, out_scale=1.0,
                 stash=None):
    """x: float32 streams [T, S, D].  pending: None or (y, scale, mix, write): the result y ([T, D] in bfloat16 or
    float32, or float32 planes [P, T, D] that are summed) of the sublayer before, still to be written into the
    streams as ``x'_t = sum_s mix[s, t] x_s + write[t] * y * scale`` (kept if write_x).  Then
    ``u = sum_t read[t] x'_t`` (read None: the plain sum) and ``out = layer_norm(u; gamma, beta, eps) * out_scale``
    for every row, or for the rows listed in `rows`.  stash: None or (carry [slots, D], stash [B, D], step): the
    first token of each of the step's sequences copies its sequence's carry (zeros at position 0) into stash."""
    _gpu(x, out, gamma, beta, read, rows)
    if x.dtype != torch.float32 or x.dim() != 3:
        raise KernelError("streams_norm: the streams are float32 [T, S, D]")
    T, S, D = x.shape
    _contig("x", x); _contig("out", out)
    _f32("gamma", gamma, D); _f32("beta", beta, D)
    if read is not None:
        _f32("read", read, S)
    n_out = out.shape[0]
    if out.shape[1] != D:
        raise KernelError(f"streams_norm: out is {tuple(out.shape)}, the width is {D}")
    y = scale = mix = write = None
    planes, stride, ycode = 1, 0, 0
    if pending is not None:
        y, scale, mix, write = pending
        _gpu(y, scale, mix, write)
        _contig("y", y)
        _f32("scale", scale, D); _f32("mix", mix, S * S); _f32("write", write, S)
        if y.dim() == 3:
            if tuple(y.shape[1:]) != (T, D) or y.dtype != torch.float32:
                raise KernelError("streams_norm: partial results must be float32 [planes, T, D]")
            planes, stride = y.shape[0], T * D
        elif tuple(y.shape) != (T, D):
            raise KernelError(f"streams_norm: the pending result is {tuple(y.shape)}, expected {(T, D)}")
        ycode = _code(y)
    if rows is not None:
        _i32("rows", rows, n_out)
    elif n_out != T:
        raise KernelError("streams_norm: out needs one row per token when rows is not given")
    carry = stash_buf = step = None
    if stash is not None:
        carry, stash_buf, step = stash
        _f32("carry", carry); _f32("stash", stash_buf)
        if carry.shape[-1] != D or stash_buf.shape != (step.n_seqs, D) or rows is not None:
            raise KernelError("streams_norm: the stash is [sequences, D], the carry [slots, D], and all rows run")
    _call("blm_streams_norm", x.data_ptr(), S, _ptr(y), ycode, planes, stride, _ptr(scale), _ptr(mix), _ptr(write),
          _ptr(read), gamma.data_ptr(), beta.data_ptr(), out.data_ptr(), _code(out), _ptr(rows), n_out, D, float(eps),
          float(out_scale), 1 if write_x else 0, _ptr(carry), _ptr(stash_buf),
          step.token_seq.data_ptr() if step else 0, step.cu_seqlens.data_ptr() if step else 0,
          step.seq_slots.data_ptr() if step else 0, step.positions.data_ptr() if step else 0, _stream())
    return out


def token_shift(n, mu, stash, carry, out, step):
    """out[t] = n[t] + (prev - n[t]) * mu with prev = n[t - 1] inside a sequence's tokens of this step and
    stash[sequence] for its first; the last token of a sequence leaves n[t] in carry[slot]."""
    _gpu(n, mu, stash, carry, out)
    T, D = n.shape
    _f32("n", n); _f32("mu", mu, D); _f32("stash", stash, step.n_seqs * D); _f32("carry", carry)
    _contig("out", out)
    if tuple(out.shape) != (T, D) or carry.shape[-1] != D or T != step.n_tokens:
        raise KernelError("token_shift: shapes do not fit")
    _call("blm_token_shift", n.data_ptr(), mu.data_ptr(), stash.data_ptr(), carry.data_ptr(), out.data_ptr(), _code(out),
          step.token_seq.data_ptr(), step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), T, D, _stream())
    return out


def xielu(z, out, a_pos, a_neg):
    """z > 0: a_pos z^2 + z/2; else a_neg (exp(z) - 1 - z) + z/2, element by element."""
    _gpu(z, out)
    _contig("z", z); _contig("out", out)
    if z.shape != out.shape or z.dtype != out.dtype:
        raise KernelError("xielu: input and output must agree in shape and dtype")
    _call("blm_xielu", z.data_ptr(), out.data_ptr(), _code(z), z.numel(), float(a_pos), float(a_neg), _stream())
    return out


# ------------------------------------------------------------------------------------------
# attention over a shared latent
def latent_write(down, q, norm_w, eps, cos_sin, rot, qabs, kcache, step, block_table, page_size, H, dn, R, Dr,
                 write_kv=True, vcache=None, adjacent=False):
    """down [T, >= R + Dr]: latent lanes then the shared key lanes; q [T, H * (dn + Dr)].  The latent is RMS-normed
    (norm_w, eps), the first `rot` of the Dr key lanes are turned by the token's position (pairs half of rot
    apart, or adjacent lanes 2i and 2i + 1; cos_sin float32 [positions, n, 2]), and the row [latent | key lanes] goes into the token's place of the
    key pages [pages, 1, page, R + Dr].  The queries' Dr lanes are turned alike into qabs[:, :, R:] (float32
    [T, H, R + Dr], or the cache's dtype).  vcache: pages [pages, 1, R, page] that get the latent transposed."""
    _gpu(down, q, norm_w, cos_sin, qabs, kcache, block_table, vcache)
    T = q.shape[0]
    _contig("cos_sin", cos_sin); _contig("kcache", kcache); _contig("qabs", qabs)
    _f32("norm_w", norm_w, R)
    if qabs.numel() != T * H * (R + Dr) or qabs.dtype not in (torch.float32, kcache.dtype):
        raise KernelError("latent_write: qabs is [T, H, R + Dr] in float32 or the cache's dtype")
    if vcache is not None:
        _contig("vcache", vcache)
        if tuple(vcache.shape) != (kcache.shape[0], 1, R, page_size) or vcache.dtype != kcache.dtype:
            raise KernelError(f"latent_write: transposed latent pages {tuple(vcache.shape)} do not fit")
    if down is None:
        if write_kv:
            raise KernelError("latent_write: rows to write need the down-projection's output")
        down, ld_down = q, max(q.stride(0), R + Dr)      # never read
    else:
        ld_down = down.stride(0)
    if down.stride(1) != 1 or q.stride(1) != 1 or down.dtype != q.dtype or kcache.dtype != q.dtype:
        raise KernelError("latent_write: down, q and the cache must share a dtype, rows contiguous")
    if tuple(q.shape) != (T, H * (dn + Dr)) or tuple(kcache.shape[1:]) != (1, page_size, R + Dr):
        raise KernelError(f"latent_write: q {tuple(q.shape)} / key pages {tuple(kcache.shape)} do not fit")
    if cos_sin.dtype != torch.float32 or cos_sin.dim() != 3 or cos_sin.shape[2] != 2 or cos_sin.shape[0] <= step.max_position:
        raise KernelError("latent_write: cos_sin must be float32 [positions, pairs, 2] and cover the step's positions")
    _i32("block_table", block_table)
    _call("blm_latent_write", down.data_ptr(), ld_down, q.data_ptr(), q.stride(0), _code(q), T, H, dn, norm_w.data_ptr(),
          float(eps), cos_sin.data_ptr(), cos_sin.shape[1], rot, qabs.data_ptr(), _code(qabs), kcache.data_ptr(),
          _ptr(vcache), step.positions.data_ptr(), step.token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], page_size,
          R, Dr, 1 if write_kv else 0, 1 if adjacent else 0, _stream())


def rmsnorm_rows(x, w, eps, out):
    """out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * w over the N lanes of out's rows; x [T, N] with any row stride (a
    slice of a projection's rows), out [T, N] contiguous in x's dtype, w float32 [N]."""
    _gpu(x, w, out)
    T, N = out.shape
    _contig("out", out); _f32("w", w, N)
    if tuple(x.shape) != (T, N) or x.stride(1) != 1 or x.dtype != out.dtype:
        raise KernelError("rmsnorm_rows: x is [T, N] with contiguous rows in out's dtype")
    _call("blm_rmsnorm_rows", x.data_ptr(), x.stride(0), _code(x), w.data_ptr(), float(eps), out.data_ptr(), T, N, _stream())
    return out


def head_project(x, in_head, w, out, out_head, K=None):
    """out[t, h * out_head + n] = sum_k x[t, h * in_head + k] * w[h, n, k] for k < K (default in_head), float
    accumulation.  x, out: 2-D with contiguous rows (any row stride); w [H, N, K] contiguous."""
    _gpu(x, w, out)
    _contig("w", w)
    H, N, Kw = w.shape
    K = Kw if K is None else K
    if K != Kw or x.stride(1) != 1 or out.stride(1) != 1 or x.shape[0] != out.shape[0]:
        raise KernelError("head_project: shapes do not fit")
    if (H - 1) * in_head + K > x.shape[1] or (H - 1) * out_head + N > out.shape[1]:
        raise KernelError("head_project: heads reach past the rows")
    _call("blm_head_project", x.data_ptr(), _code(x), x.stride(0), in_head, w.data_ptr(), _code(w), out.data_ptr(),
          _code(out), out.stride(0), out_head, x.shape[0], H, N, K, _stream())
    return out


_latent_scratch = {}
LATENT_SCRATCH_FLOATS = 1 << 23


def latent_attn_init(device):
    """The workspace of the split form (partial results of the pieces), one per device and of a fixed size, so
    that a recorded launch's address stays good.  The first call for a device must come before any recording."""
    device = torch.device(device)
    key = device.index if device.index is not None else torch.cuda.current_device()
    buf = _latent_scratch.get(key)
    if buf is None:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("latent_attn_init: the first call for a device must come before any graph capture")
        buf = _latent_scratch[key] = torch.empty(LATENT_SCRATCH_FLOATS, dtype=torch.float32, device=torch.device("cuda", key))
    return buf


def latent_attn_max_splits(T, H, R):
    """Most pieces a (token, head)'s rows can be cut into for T tokens."""
    if T * H > ARRIVAL_COUNTERS:
        return 1
    return max(1, LATENT_SCRATCH_FLOATS // (T * H * (R + 2)))



def latent_attn(qabs, olat, kcache, step, block_table, page_size, H, R, Dr, scale, n_splits=1):
    """softmax over each query's visible rows of (qabs . [latent | key lanes]) * scale, times the latents:
    olat float32 [T, H, R].  qabs float32 [T, H, R + Dr]; kcache [pages, 1, page, R + Dr]."""
    _gpu(qabs, olat, kcache, block_table)
    T = qabs.shape[0]
    _f32("qabs", qabs, T * H * (R + Dr)); _f32("olat", olat, T * H * R)
    _contig("kcache", kcache); _i32("block_table", block_table)
    if tuple(kcache.shape[1:]) != (1, page_size, R + Dr):
        raise KernelError(f"latent_attn: key pages {tuple(kcache.shape)} do not fit rows of {R + Dr}")
    part_o = part_ml = arrivals = None
    if n_splits > 1:
        need = T * H * n_splits * (R + 2)
        if n_splits > latent_attn_max_splits(T, H, R):
            raise KernelError("latent_attn: more pieces than the workspace holds (see latent_attn_max_splits)")
        buf = latent_attn_init(qabs.device)
        part_o, part_ml = buf[: T * H * n_splits * R], buf[T * H * n_splits * R: need]
        arrivals = arrival_counters(qabs.device)
    _call("blm_latent_attn", qabs.data_ptr(), olat.data_ptr(), _code(kcache), step.positions.data_ptr(),
          step.token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], kcache.data_ptr(), page_size, T, H, R,
          Dr, float(scale), n_splits, _ptr(part_o), _ptr(part_ml), _ptr(arrivals), _stream())
    return olat


def latent_attn_mfma_supported(dtype, R, Dr, page_size=64):
    return dtype == torch.bfloat16 and page_size == 64 and bool(library().blm_latent_attn_mfma_supported(R, Dr))


def latent_attn_mfma_max_splits(n_seqs, max_new, H, R):
    """Most pieces the matrix-core form can cut the pages into for a step of this shape."""
    waves = n_seqs * ((max_new * H + 15) // 16)
    return max(1, LATENT_SCRATCH_FLOATS // (waves * 16 * (R + 2)))


def latent_attn_mfma(q, olat, kcache, vcache, step, block_table, page_size, H, R, Dr, scale, n_splits=1):
    """The same function as latent_attn on the matrix cores: q bfloat16 [T, H, R + Dr], key pages and transposed
    latent pages ([pages, 1, R, 64]) in bfloat16; olat float32 [T, H, R]."""
    _gpu(q, olat, kcache, vcache, block_table)
    T = q.shape[0]
    _contig("q", q); _contig("kcache", kcache); _contig("vcache", vcache); _i32("block_table", block_table)
    _f32("olat", olat, T * H * R)
    if q.dtype != torch.bfloat16 or kcache.dtype != torch.bfloat16 or vcache.dtype != torch.bfloat16 or q.numel() != T * H * (R + Dr):
        raise KernelError("latent_attn_mfma: queries [T, H, R + Dr] and both kinds of pages in bfloat16")
    if tuple(kcache.shape[1:]) != (1, page_size, R + Dr) or tuple(vcache.shape) != (kcache.shape[0], 1, R, page_size):
        raise KernelError(f"latent_attn_mfma: pages {tuple(kcache.shape)} / {tuple(vcache.shape)} do not fit")
    if T != step.n_tokens or step.cu_seqlens.numel() < step.n_seqs + 1 or block_table.shape[0] < step.n_seqs:
        raise KernelError("latent_attn_mfma: the step's index arrays do not fit the queries")
    part_o = part_ml = None
    if n_splits > 1:
        if n_splits > latent_attn_mfma_max_splits(step.n_seqs, step.max_new, H, R):
            raise KernelError("latent_attn_mfma: more pieces than the workspace holds (see latent_attn_mfma_max_splits)")
        cols = step.n_seqs * ((step.max_new * H + 15) // 16) * 16
        buf = latent_attn_init(q.device)
        part_o, part_ml = buf[: cols * n_splits * R], buf[cols * n_splits * R: cols * n_splits * (R + 2)]
    _call("blm_latent_attn_mfma", q.data_ptr(), olat.data_ptr(), step.cu_seqlens.data_ptr(), step.lens_after.data_ptr(),
          block_table.data_ptr(), block_table.shape[1], kcache.data_ptr(), vcache.data_ptr(), page_size, step.n_seqs,
          step.max_new, H, R, Dr, float(scale), n_splits, _ptr(part_o), _ptr(part_ml), _stream())
    return olat


# ------------------------------------------------------------------------------------------
# recurrent mixers
def hgrn2_scan(proj, f_bias, low, norm_w, eps, state, o_raw, out, step, H, dk, dv):
    """proj [T, >= 2 H dk + H dv]: queries, forget-gate logits, values.  state float32 [slots, H, dk, dv] is read
    and left updated for the step's sequences; o_raw: zeroed float32 [T, H * dv] for the unnormalised results;
    out [T, H * dv] in proj's dtype."""
    _gpu(proj, f_bias, low, norm_w, state, o_raw, out)
    _f32("o_raw", o_raw, proj.shape[0] * H * dv)
    gates = torch.empty(proj.shape[0], 2 * H * dk, dtype=torch.float32, device=proj.device)
    _f32("f_bias", f_bias, H * dk); _f32("low", low, H * dk); _f32("norm_w", norm_w, dv); _f32("state", state)
    _contig("out", out)
    if proj.stride(1) != 1 or out.dtype != proj.dtype or tuple(out.shape) != (proj.shape[0], H * dv) \
            or tuple(state.shape[1:]) != (H, dk, dv):
        raise KernelError("hgrn2_scan: shapes do not fit")
    _call("blm_hgrn2_scan", proj.data_ptr(), _code(proj), proj.stride(0), f_bias.data_ptr(), low.data_ptr(),
          norm_w.data_ptr(), float(eps), state.data_ptr(), gates.data_ptr(), o_raw.data_ptr(), out.data_ptr(),
          step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), proj.shape[0], step.n_seqs, H, dk, dv, _stream())
    return out


def conv_prepare(proj, taps_w, hist, out, step, C, G, dk):
    """Causal convolution per channel over the first C columns of proj ([q: G dk | k: G dk | v]) with SiLU, unit
    norms of the q and k heads (q also times dk^-1/2) -> out float32 [T, C]; hist float32 [slots, taps - 1, C] is
    read and then left holding each sequence's last taps - 1 inputs."""
    _gpu(proj, taps_w, hist, out)
    T = proj.shape[0]
    taps = taps_w.shape[1]
    _f32("taps_w", taps_w, C * taps); _f32("hist", hist); _f32("out", out, T * C)
    if proj.stride(1) != 1 or proj.shape[1] < C or (taps > 1 and tuple(hist.shape[1:]) != (taps - 1, C)):
        raise KernelError("conv_prepare: shapes do not fit")
    _call("blm_conv_prepare", proj.data_ptr(), _code(proj), proj.stride(0), taps_w.data_ptr(), taps, hist.data_ptr(),
          out.data_ptr(), step.token_seq.data_ptr(), step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), T, step.n_seqs,
          C, G, dk, _stream())
    return out


def delta_scan(qkv, beta_src, beta_col, decay_in, dt_bias, a_log, gate_in, norm_w, eps, state, o_raw, out, step, H, G,
               dk, dv):
    """The delta rule with a decay per key channel over conv_prepare's rows; see the kernel for the formulas.
    beta_src: the tensor whose column beta_col + h holds head h's write-strength logit; decay_in [T, H dk] and
    gate_in [T, H dv] in the same dtype; o_raw: zeroed float32 [T, H * dv]; out [T, H * dv] in that dtype."""
    _gpu(qkv, beta_src, decay_in, dt_bias, a_log, gate_in, norm_w, state, o_raw, out)
    T, C = qkv.shape
    _f32("o_raw", o_raw, T * H * dv)
    gates = torch.empty(T, H * dk + H, dtype=torch.float32, device=qkv.device)
    _f32("qkv", qkv); _f32("dt_bias", dt_bias, H * dk); _f32("a_log", a_log, H); _f32("norm_w", norm_w, dv)
    _f32("state", state)
    _contig("decay_in", decay_in); _contig("gate_in", gate_in); _contig("out", out)
    if not (beta_src.dtype == decay_in.dtype == gate_in.dtype == out.dtype) or beta_src.stride(1) != 1:
        raise KernelError("delta_scan: the projections and the output must share a dtype")
    if tuple(decay_in.shape) != (T, H * dk) or tuple(gate_in.shape) != (T, H * dv) or tuple(out.shape) != (T, H * dv) \
            or tuple(state.shape[1:]) != (H, dk, dv) or beta_col + H > beta_src.shape[1]:
        raise KernelError("delta_scan: shapes do not fit")
    _call("blm_delta_scan", qkv.data_ptr(), C, beta_src.data_ptr(), _code(out), beta_src.stride(0), beta_col,
          decay_in.data_ptr(), dt_bias.data_ptr(), a_log.data_ptr(), gate_in.data_ptr(), norm_w.data_ptr(), float(eps),
          state.data_ptr(), gates.data_ptr(), o_raw.data_ptr(), out.data_ptr(), step.cu_seqlens.data_ptr(),
          step.seq_slots.data_ptr(), T, step.n_seqs, H, G, dk, dv, _stream())
    return out


# ------------------------------------------------------------------------------------------
# layers whose sublayers run side by side: input convolution, residual add, side input, clamped and routed gating
def _planes(who, y, T, D):
    """(planes, dtype code) of a sublayer's result: [T, D], or float32 planes [P, T, D]."""
    _contig(who, y)
    if y.dim() == 3:
        if tuple(y.shape[1:]) != (T, D) or y.dtype != torch.float32:
            raise KernelError(f"{who}: partial results must be float32 [planes, {T}, {D}], got {tuple(y.shape)}")
        return y.shape[0], 0
    if tuple(y.shape) != (T, D):
        raise KernelError(f"{who}: expected [{T}, {D}], got {tuple(y.shape)}")
    return 1, _code(y)


def input_conv(n, hist, weights, outs, step):
    """outs[r][t] = n[t] + causal convolution of n's rows with weights[r] ([D, taps] float32) for one or two readers
    of the same rows n (float32 [T, D]); rows before the step come from hist (float32 [slots, taps - 1, D]), which
    is then left holding each sequence's last taps - 1 rows."""
    _gpu(n, hist, *weights, *outs)
    T, D = n.shape
    _f32("n", n)
    taps = weights[0].shape[1]
    if not 1 <= len(weights) <= 2 or len(outs) != len(weights) or T != step.n_tokens:
        raise KernelError("input_conv: one or two readers, an output for each, one row per token of the step")
    for w, o in zip(weights, outs):
        _f32("weights", w, D * taps); _contig("out", o)
        if tuple(o.shape) != (T, D) or o.dtype != outs[0].dtype:
            raise KernelError("input_conv: outputs are [T, D] of one dtype")
    if taps > 1:
        _f32("hist", hist)
        if tuple(hist.shape[1:]) != (taps - 1, D):
            raise KernelError(f"input_conv: the history is {tuple(hist.shape)}, expected [slots, {taps - 1}, {D}]")
    two = len(weights) == 2
    _call("blm_input_conv", n.data_ptr(), _ptr(hist) if taps > 1 else 0, weights[0].data_ptr(),
          weights[1].data_ptr() if two else 0, outs[0].data_ptr(), outs[1].data_ptr() if two else 0, len(weights),
          _code(outs[0]), taps, step.token_seq.data_ptr(), step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), T,
          step.n_seqs, D, _stream())
    return outs


def residual_add(h, a, b=None, bias=None, copy=None):
    """h += a (+ b) (+ bias) in float32; copy (if given, [T, D] in any kernel dtype) receives the new h.  a, b: [T, D]
    or float32 planes [P, T, D]."""
    _gpu(h, a, b, bias, copy)
    T, D = h.shape
    _f32("h", h)
    pa, ca = _planes("residual_add: a", a, T, D)
    pb, cb = _planes("residual_add: b", b, T, D) if b is not None else (1, 0)
    if bias is not None:
        _f32("bias", bias, D)
    if copy is not None:
        _contig("copy", copy)
        if tuple(copy.shape) != (T, D):
            raise KernelError("residual_add: the copy is [T, D]")
    _call("blm_residual_add", h.data_ptr(), a.data_ptr(), ca, pa, _ptr(b), cb, pb, _ptr(bias), _ptr(copy),
          _code(copy) if copy is not None else 0, T, D, _stream())
    return h


def side_gate(z, table, col0, ids, out, token_source=None):
    """out[t, j] = gelu_tanh(z[t, j]) * table[token of t, col0 + j]; token_source: None or the step's (rows, cell) of
    tokens that are still on the device (see embed_gather_from)."""
    _gpu(z, table, ids, out)
    T, dim = z.shape
    _contig("z", z); _contig("table", table); _contig("out", out)
    _i32("ids", ids, T)
    if out.shape != z.shape or out.dtype != z.dtype or table.dim() != 2:
        raise KernelError("side_gate: shapes do not fit")
    rows = cell = None
    if token_source is not None:
        rows, cell = token_source
        _i32("source_rows", rows, T)
        if cell.dtype != torch.int64 or cell.numel() != 1:
            raise KernelError("side_gate: the cell is one int64 on the device")
    _call("blm_side_gate", z.data_ptr(), _code(z), table.data_ptr(), _code(table), table.shape[1], int(col0), ids.data_ptr(),
          _ptr(rows), _ptr(cell), table.shape[0], out.data_ptr(), T, dim, _stream())
    return out


def rms_scale(y, w, eps, out):
    """out = y / sqrt(mean(y^2) + eps) * w as float32 [T, D]; y: [T, D] or float32 planes [P, T, D]."""
    _gpu(y, w, out)
    T, D = out.shape
    _f32("out", out); _f32("w", w, D)
    planes, code = _planes("rms_scale: y", y, T, D)
    _call("blm_rms_scale", y.data_ptr(), code, planes, w.data_ptr(), out.data_ptr(), T, D, float(eps), _stream())
    return out


def clamped_glu(gate_up, out, limit, alpha):
    """g = min(gate, limit), u = clamp(up, -limit, limit): out = g * sigmoid(alpha * g) * (u + 1); gate_up [T, 2 I]."""
    _gpu(gate_up, out)
    T, I = out.shape
    _contig("gate_up", gate_up); _contig("out", out)
    if tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError("clamped_glu: gate_up is [T, 2 I] in out's dtype")
    _call("blm_clamped_glu", gate_up.data_ptr(), out.data_ptr(), _code(out), T, I, float(limit), float(alpha), _stream())
    return out


def gelu_glu(gate_up, out):
    """out = gelu_tanh(gate) * up; gate_up [T, 2 I]: gate columns, then up columns."""
    _gpu(gate_up, out)
    T, I = out.shape
    _contig("gate_up", gate_up); _contig("out", out)
    if tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError("gelu_glu: gate_up is [T, 2 I] in out's dtype")
    _call("blm_gelu_glu", gate_up.data_ptr(), out.data_ptr(), _code(out), T, I, _stream())
    return out


def softcap(logits, cap):
    """logits <- cap * tanh(logits / cap), in place on contiguous float32."""
    _gpu(logits)
    _contig("logits", logits)
    if logits.dtype != torch.float32 or not cap > 0:
        raise KernelError("softcap: float32 logits and a positive cap")
    _call("blm_softcap", logits.data_ptr(), logits.numel(), float(cap), _stream())
    return logits


def sigmoid_gate(x, gate):
    """x[t, c] *= sigmoid(gate[t, c]) in place; x [T, N] and gate [T, N] with contiguous rows of any stride, one dtype."""
    _gpu(x, gate)
    T, N = x.shape
    if tuple(gate.shape) != (T, N) or x.stride(1) != 1 or gate.stride(1) != 1 or x.dtype != gate.dtype:
        raise KernelError("sigmoid_gate: x and gate are [T, N] with contiguous rows in one dtype")
    _call("blm_sigmoid_gate", x.data_ptr(), x.stride(0), gate.data_ptr(), gate.stride(0), _code(x), T, N, _stream())
    return x


def moe_route(logits, bias, n_experts, top, shared_col, weights):
    """weights [T, E + 1] float32: for each token the softmax over its `top` largest of (logits[:, :E] + bias) at the
    chosen experts' places and zero elsewhere; at E the sigmoid of logits[:, shared_col] (shared_col < 0: one)."""
    _gpu(logits, bias, weights)
    T = logits.shape[0]
    _f32("logits", logits); _f32("bias", bias, n_experts); _f32("weights", weights, T * (n_experts + 1))
    _call("blm_moe_route", logits.data_ptr(), logits.shape[1], bias.data_ptr(), n_experts, top, shared_col,
          weights.data_ptr(), T, _stream())
    return weights


def moe_gate(gate_up, weights, out, n_experts, expert_inner):
    """out[t, i] = silu(gate) * up * weights[t, expert of column i] for experts stacked along the columns (expert e at
    columns e * expert_inner, a shared expert behind them with the weight at E); gate_up [T, 2 I], out [T, I]."""
    _gpu(gate_up, weights, out)
    T, I = out.shape
    _contig("gate_up", gate_up); _contig("out", out)
    _f32("weights", weights, T * (n_experts + 1))
    if tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError("moe_gate: gate_up is [T, 2 I] in out's dtype")
    _call("blm_moe_gate", gate_up.data_ptr(), weights.data_ptr(), out.data_ptr(), _code(out), T, I, n_experts,
          expert_inner, _stream())
    return out


def moe_route_grouped(logits, correction, n_experts, n_identity, groups, keep, top, weights):
    """weights [T, E + 1] float32 from logits [T, >= E + n_identity] float32: scores are the softmax over all E + n_identity
    logits; the choice goes by score + correction (None: the score) among the experts of the `keep` best of `groups`
    equal groups of neighbours (a group's rank: its largest choice; groups <= 1: among all); the `top` chosen experts'
    weights are their scores over the sum of the chosen scores.  Column e < E: expert e's weight or zero; column E: the
    weights of the chosen ones among the last n_identity (experts that pass their input through), added up."""
    _gpu(logits, correction, weights)
    T = logits.shape[0]
    _f32("logits", logits); _f32("weights", weights, T * (n_experts + 1))
    if correction is not None:
        _f32("correction", correction, n_experts + n_identity)
    if logits.dim() != 2 or tuple(weights.shape) != (T, n_experts + 1):
        raise KernelError("moe_route_grouped: logits [T, N], weights [T, E + 1]")
    _call("blm_moe_route_grouped", logits.data_ptr(), logits.shape[1], _ptr(correction), int(n_experts), int(n_identity),
          int(groups), int(keep), int(top), weights.data_ptr(), T, _stream())
    return weights


MAX_ADD_TERMS = 4


def scaled_add(h, terms):
    """h[t, c] += sum over terms (y, chan, row) of chan[c] * row[t] * y[t, c] in float32.  y: [T, D] in a kernel dtype or
    float32 planes [P, T, D] (summed); chan: float32 [D] or None (one); row: float32 [T] (any stride) or None (one)."""
    T, D = h.shape
    _f32("h", h)
    if not 1 <= len(terms) <= MAX_ADD_TERMS:
        raise KernelError(f"scaled_add: one to {MAX_ADD_TERMS} terms, got {len(terms)}")
    args = []
    for y, chan, row in terms:
        _gpu(y, chan, row)
        planes, code = _planes("scaled_add: y", y, T, D)
        if chan is not None:
            _f32("chan", chan, D)
        ld = 0
        if row is not None:
            if row.dtype != torch.float32 or row.dim() != 1 or row.shape[0] != T:
                raise KernelError("scaled_add: a row coefficient is float32 [T]")
            ld = row.stride(0) if T > 1 else 1
            if ld < 1:
                raise KernelError("scaled_add: a row coefficient's stride must be positive")
        args += [y.data_ptr(), code, planes, _ptr(chan), _ptr(row), ld]
    args += [0, 0, 0, 0, 0, 0] * (MAX_ADD_TERMS - len(terms))
    _call("blm_scaled_add", h.data_ptr(), T, D, len(terms), *args, _stream())
    return h


def gla_segments(step, H, dv, compute_units=256):
    """(segments, tokens per segment) into which gla_scan cuts the sequences of a step: prompts are walked by several
    wavefronts at once, each over a stretch of at least 64 tokens (a multiple of 8), as many as give every compute
    unit about thirty-two wavefronts; steps of few tokens per sequence are not cut."""
    if step.n_tokens <= 4 * step.n_seqs or step.max_new < 128 or dv > 256:
        return 1, 0
    walkers = step.n_seqs * H * ((dv + 3) // 4)
    n_seg = max(1, min(step.max_new // 64, (32 * compute_units) // max(1, walkers)))
    if n_seg == 1:
        return 1, 0
    seg_len = (-(-step.max_new // n_seg) + 7) // 8 * 8
    return -(-step.max_new // seg_len), seg_len


GATE_MODES = {"sigmoid": 1, "silu": 2}


def gla_scan(proj, decay_in, decay_bias, tau, norm_w, eps, state, o_raw, out, step, H, dk, dv, segments=None,
             fixed_decay=None, activation=None, q_scale=None, norm_all=False, gate="silu"):
    """Gated linear attention over proj [T, >= 2 H dk + 2 H dv]: queries, keys, values, output-gate logits;
    decay_in [T, H dk]: the decays' logits before their bias.  state float32 [slots, H, dk, dv] is read and left
    updated; o_raw: zeroed float32 [T, H * dv]; out [T, H * dv] in proj's dtype.  segments: (count, tokens each) as
    gla_segments gives them (the default), or (1, 0) for one walk per sequence.
    The same recurrence with other surroundings: fixed_decay (float32 [H * dk]): the decays of every token, in place of
    decay_in, decay_bias and tau (which are then None); activation "silu": on queries, keys and values, rounded to
    proj's dtype (where the sequences are walked in segments, proj's first columns are activated in place); q_scale: the
    queries' factor (default dk^-1/2); norm_all: one root mean square over all heads' lanes, norm_w [H * dv] (default:
    per head, norm_w [dv]); gate: "silu" or "sigmoid" of the output gate's logits."""
    _gpu(proj, decay_in, decay_bias, norm_w, state, o_raw, out, fixed_decay)
    T = proj.shape[0]
    _f32("o_raw", o_raw, T * H * dv); _f32("norm_w", norm_w, H * dv if norm_all else dv); _f32("state", state)
    _contig("out", out)
    if activation not in (None, "silu") or gate not in GATE_MODES:
        raise KernelError(f"gla_scan: activation {activation!r} or gate {gate!r} unknown")
    if proj.stride(1) != 1 or out.dtype != proj.dtype or tuple(out.shape) != (T, H * dv) or tuple(state.shape[1:]) != (H, dk, dv) \
            or proj.shape[1] < 2 * H * dk + 2 * H * dv or T != step.n_tokens:
        raise KernelError("gla_scan: shapes do not fit")
    gates = None
    if fixed_decay is not None:
        _f32("fixed_decay", fixed_decay, H * dk)
        if decay_in is not None or decay_bias is not None:
            raise KernelError("gla_scan: fixed decays come without decay logits")
    else:
        _f32("decay_bias", decay_bias, H * dk); _contig("decay_in", decay_in)
        if decay_in.dtype != proj.dtype or tuple(decay_in.shape) != (T, H * dk):
            raise KernelError("gla_scan: shapes do not fit")
        gates = torch.empty(T, H * dk, dtype=torch.float32, device=proj.device)
    n_seg, seg_len = segments if segments is not None else gla_segments(step, H, dv)
    seg_end = seg_start = seg_decay = q_tilde = None
    if n_seg > 1:
        B = step.n_seqs
        seg_end = torch.empty(B, n_seg, H, dk, dv, dtype=torch.float32, device=proj.device)
        seg_start = torch.empty_like(seg_end)
        seg_decay = torch.empty(B, n_seg, H, dk, dtype=torch.float32, device=proj.device)
        q_tilde = torch.empty(T, H, dk, dtype=torch.float32, device=proj.device)
    _call("blm_gla_scan", proj.data_ptr(), _code(proj), proj.stride(0), _ptr(decay_in), _ptr(decay_bias),
          float(tau) if tau is not None else 0.0, norm_w.data_ptr(), float(eps), state.data_ptr(), _ptr(gates), o_raw.data_ptr(),
          out.data_ptr(), step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), T, step.n_seqs, H, dk, dv, step.max_new, n_seg,
          seg_len, _ptr(seg_end), _ptr(seg_start), _ptr(seg_decay), _ptr(q_tilde), _ptr(fixed_decay),
          1 if activation == "silu" else 0, float(q_scale) if q_scale is not None else 0.0, 1 if norm_all else 0,
          GATE_MODES[gate], _stream())
    return out


LIGHTNING_CHUNK = 64
_lc_ready = set()


def lightning_chunks_init(device=None):
    """Once per device, outside any stream capture, before the first lightning_chunks (its kernels take more shared
    memory than a kernel gets without asking)."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _lc_ready:
        with torch.cuda.device(index):
            _call("blm_lightning_chunks_init")
        _lc_ready.add(index)


def lightning_chunks_supported(dk, dv):
    return bool(library().blm_lightning_chunks_supported(int(dk), int(dv)))


def decay_powers(decays, device):
    """float32 [heads, 65]: powers 0 .. 64 of every head's decay, from double precision."""
    a = torch.tensor([float(x) for x in decays], dtype=torch.float64).reshape(-1, 1)
    return (a ** torch.arange(LIGHTNING_CHUNK + 1, dtype=torch.float64)).to(torch.float32).contiguous().to(device)


def lightning_chunks(proj, powers, norm_w, eps, state, o_raw, out, step, H, dk, dv, activation=None, norm_all=False,
                     gate="sigmoid"):
    """Linear attention with one constant decay per head over the prompts of a step, in chunks of 64 tokens as float32
    matrix products: proj [T, >= 2 H dk + 2 H dv] (queries, keys, values, output-gate logits), powers as
    decay_powers gives them, state float32 [slots, H, dk, dv] read and left updated, o_raw float32 [T, H * dv], out
    [T, H * dv] in proj's dtype.  activation ("silu": proj's queries, keys and values are activated in place), norm_all,
    gate as for gla_scan; the queries have no factor."""
    _gpu(proj, powers, norm_w, state, o_raw, out)
    T = proj.shape[0]
    _f32("o_raw", o_raw, T * H * dv); _f32("norm_w", norm_w, H * dv if norm_all else dv); _f32("state", state)
    _f32("powers", powers, H * (LIGHTNING_CHUNK + 1)); _contig("out", out)
    if activation not in (None, "silu") or gate not in GATE_MODES:
        raise KernelError(f"lightning_chunks: activation {activation!r} or gate {gate!r} unknown")
    if proj.stride(1) != 1 or out.dtype != proj.dtype or tuple(out.shape) != (T, H * dv) or tuple(state.shape[1:]) != (H, dk, dv) \
            or proj.shape[1] < 2 * H * dk + 2 * H * dv or T != step.n_tokens:
        raise KernelError("lightning_chunks: shapes do not fit")
    B, n_seg = step.n_seqs, -(-step.max_new // LIGHTNING_CHUNK)
    seg_end = torch.empty(B, n_seg, H, dk, dv, dtype=torch.float32, device=proj.device)
    seg_start = torch.empty_like(seg_end)
    _call("blm_lightning_chunks", proj.data_ptr(), _code(proj), proj.stride(0), powers.data_ptr(), norm_w.data_ptr(), float(eps),
          state.data_ptr(), o_raw.data_ptr(), out.data_ptr(), step.cu_seqlens.data_ptr(), step.seq_slots.data_ptr(), T, B, H, dk,
          dv, step.max_new, n_seg, seg_end.data_ptr(), seg_start.data_ptr(),
          1 if activation == "silu" else 0, 1 if norm_all else 0, GATE_MODES[gate], _stream())
    return out


def qkv_prepare(qkv, bias, cos_sin, rot, step, block_table, kcache, vcache, page_size, H, G, dk, dv, write_kv=True,
                adjacent=False, values_are_keys=False, q_scale=None):
    """Bias, rotation of the first `rot` lanes of every query and key head by the token's position (lane i with
    lane i + rot/2, or with adjacent lanes 2i and 2i + 1; cos_sin float32 [positions, >= rot/2, 2] rows of exactly
    rot/2 pairs), queries in place, rotated keys and values into the pages (key pages [pages, G, page, dk], value pages
    [pages, G, dv, page]).  write_kv False: qkv holds queries only and nothing is stored.  values_are_keys: the rows
    hold no values; a token's values are its keys as projected, before the rotation (dv = dk).  q_scale (float32 [H]
    or None): query head h is multiplied by q_scale[h] behind the rotation."""
    _gpu(qkv, bias, cos_sin, block_table, kcache, vcache, q_scale)
    if q_scale is not None:
        _f32("q_scale", q_scale, H)
    T = qkv.shape[0]
    if qkv.stride(1) != 1:
        raise KernelError("qkv_prepare: rows must be contiguous")
    if values_are_keys and dv != dk:
        raise KernelError("qkv_prepare: values that are the keys have the keys' head size")
    need = H * dk + (G * (dk + (0 if values_are_keys else dv)) if write_kv else 0)
    if qkv.shape[1] < need or T != step.n_tokens:
        raise KernelError(f"qkv_prepare: rows of {qkv.shape[1]}, needs {need}")
    if bias is not None:
        _f32("bias", bias, need)
    if rot:
        _contig("cos_sin", cos_sin)
        if cos_sin.dtype != torch.float32 or tuple(cos_sin.shape[1:]) != (rot // 2, 2) or cos_sin.shape[0] <= step.max_position:
            raise KernelError("qkv_prepare: cos_sin must be float32 [positions, rot/2, 2] and cover the step's positions")
    if write_kv:
        _contig("kcache", kcache); _contig("vcache", vcache); _i32("block_table", block_table)
        if kcache.dtype != qkv.dtype or vcache.dtype != qkv.dtype or tuple(kcache.shape[1:]) != (G, page_size, dk) \
                or tuple(vcache.shape) != (kcache.shape[0], G, dv, page_size):
            raise KernelError(f"qkv_prepare: pages {tuple(kcache.shape)} / {tuple(vcache.shape)} do not fit")
    _call("blm_qkv_prepare", qkv.data_ptr(), _code(qkv), qkv.stride(0), _ptr(bias), _ptr(cos_sin) if rot else 0, rot,
          step.positions.data_ptr(), step.token_seq.data_ptr(), _ptr(block_table) if write_kv else 0,
          block_table.shape[1] if write_kv else 0, _ptr(kcache) if write_kv else 0, _ptr(vcache) if write_kv else 0,
          page_size, T, H, G, dk, dv, 1 if write_kv else 0, 1 if adjacent else 0, 1 if values_are_keys else 0, _ptr(q_scale),
          _stream())
    return qkv


def sink_attn(q, out, sinks, mix, step, block_table, kcache, vcache, page_size, H, G, dk, dv, scale, window):
    """Attention whose softmax denominator also holds exp(sinks[h]) (sinks None: a plain softmax) and whose weights
    are mixed between heads by mix [H, H] (None: not mixed) before head h reads the values of its own key-value head.
    q [T, >= H dk] rows (queries already rotated), out [T, H * dv] in q's dtype."""
    _gpu(q, out, sinks, mix, block_table, kcache, vcache)
    T = q.shape[0]
    _contig("out", out); _contig("kcache", kcache); _contig("vcache", vcache); _i32("block_table", block_table)
    if q.stride(1) != 1 or out.dtype != q.dtype or kcache.dtype != q.dtype or vcache.dtype != q.dtype:
        raise KernelError("sink_attn: queries, pages and output share a dtype; rows contiguous")
    if tuple(out.shape) != (T, H * dv) or tuple(kcache.shape[1:]) != (G, page_size, dk) \
            or tuple(vcache.shape) != (kcache.shape[0], G, dv, page_size) or T != step.n_tokens:
        raise KernelError(f"sink_attn: shapes do not fit: out {tuple(out.shape)}, pages {tuple(kcache.shape)} / {tuple(vcache.shape)}")
    if sinks is not None:
        _f32("sinks", sinks, H)
    if mix is not None:
        _f32("mix", mix, H * H)
    A = torch.empty(T, H, G if mix is not None else 1, dv, dtype=torch.float32, device=q.device)
    _call("blm_sink_attn", q.data_ptr(), q.stride(0), out.data_ptr(), _code(q), A.data_ptr(), _ptr(sinks), _ptr(mix),
          step.positions.data_ptr(), step.token_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1],
          kcache.data_ptr(), vcache.data_ptr(), page_size, T, H, G, dk, dv, float(scale), int(window), _stream())
    return out


_sam_ready = set()


def sink_attn_mfma_init(device=None):
    """Once per device, outside any stream capture, before the first sink_attn_mfma of a prompt (the form that stages
    pages takes more shared memory than a kernel gets without asking)."""
    index = torch.device(device or "cuda").index
    index = torch.cuda.current_device() if index is None else index
    if index not in _sam_ready:
        with torch.cuda.device(index):
            _call("blm_sink_attn_mfma_init")
        _sam_ready.add(index)


def sink_attn_mfma_supported(dtype, dk, dv, page_size=64):
    return dtype == torch.bfloat16 and page_size == 64 and bool(library().blm_sink_attn_mfma_supported(int(dk), int(dv)))


def sink_attn_mfma_max_splits(n_seqs, max_new, H, G, dv, mixed):
    """Most pieces the matrix-core form can cut a tile's pages into for a step of this shape (its partial results
    live in the fixed workspace of latent_attn_init)."""
    cols = n_seqs * G * ((max_new * (H // G) + 15) // 16) * 16
    return max(1, min(64, LATENT_SCRATCH_FLOATS // (cols * ((G if mixed else 1) * dv + 2))))


def sink_attn_mfma(q, out, sinks, mix, step, block_table, kcache, vcache, page_size, H, G, dk, dv, scale, window, n_splits=1,
                   group_batch=0):
    """sink_attn on the matrix cores: bfloat16 queries, pages (64 keys) and output; the same arguments, and n_splits:
    into how many pieces every tile's pages are cut (a second kernel adds them up); group_batch: 0, or the most
    key-value heads a wavefront accumulates at a time (fewer: more wavefronts, each with less to wait for)."""
    _gpu(q, out, sinks, mix, block_table, kcache, vcache)
    sink_attn_mfma_init(q.device)
    T = q.shape[0]
    _contig("out", out); _contig("kcache", kcache); _contig("vcache", vcache); _i32("block_table", block_table)
    if q.stride(1) != 1 or not (q.dtype == out.dtype == kcache.dtype == vcache.dtype == torch.bfloat16):
        raise KernelError("sink_attn_mfma: queries, pages and output in bfloat16; rows contiguous")
    if tuple(out.shape) != (T, H * dv) or tuple(kcache.shape[1:]) != (G, page_size, dk) \
            or tuple(vcache.shape) != (kcache.shape[0], G, dv, page_size) or T != step.n_tokens \
            or block_table.shape[0] < step.n_seqs or step.cu_seqlens.numel() < step.n_seqs + 1:
        raise KernelError(f"sink_attn_mfma: shapes do not fit: out {tuple(out.shape)}, pages {tuple(kcache.shape)} / {tuple(vcache.shape)}")
    if sinks is not None:
        _f32("sinks", sinks, H)
    if mix is not None:
        _f32("mix", mix, H * H)
    n_out = G if mix is not None else 1
    A = torch.empty(T, H, n_out, dv, dtype=torch.float32, device=q.device)
    part_o = part_ml = None
    if n_splits > 1:
        if n_splits > sink_attn_mfma_max_splits(step.n_seqs, step.max_new, H, G, dv, mix is not None):
            raise KernelError("sink_attn_mfma: more pieces than the workspace holds (see sink_attn_mfma_max_splits)")
        cols = step.n_seqs * G * ((step.max_new * (H // G) + 15) // 16) * 16
        buf = latent_attn_init(q.device)
        part_o, part_ml = buf[: cols * n_splits * n_out * dv], buf[cols * n_splits * n_out * dv: cols * n_splits * (n_out * dv + 2)]
    _call("blm_sink_attn_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), A.data_ptr(), _ptr(sinks), _ptr(mix),
          step.token_seq.data_ptr(), step.cu_seqlens.data_ptr(), step.lens_after.data_ptr(), block_table.data_ptr(),
          block_table.shape[1], kcache.data_ptr(), vcache.data_ptr(), page_size, step.n_seqs, step.max_new, T, H, G, dk, dv,
          float(scale), int(window), int(n_splits), int(group_batch), _ptr(part_o), _ptr(part_ml), _stream())
    return out
