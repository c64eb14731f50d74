"""Python face of the HIP kernel library: loads ``libburnlm_hip.so`` through ctypes and wraps
each entry point with checks of device, dtype, shape and contiguity.  Kernels run on torch's
current HIP stream.  There is no fallback: without the library, or off the GPU, calls raise."""
from __future__ import annotations

import ctypes
import threading

import torch

from . import build as _build

ABI_VERSION = 24
_lib = None
_lock = threading.Lock()

_c_int, _c_float, _c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_void_p


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


_SIGNATURES = {
    "blm_embed_gather": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "blm_embed_gather_from": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                              _c_void_p],
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
                        _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    "blm_attn_decode_supported": [_c_int, _c_int, _c_int],
    "blm_attn_prefill_mfma_supported": [_c_int, _c_int, _c_int],
    "blm_attn_prefill_mfma": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int,
                              _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                              _c_int, _c_int, _c_void_p],
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
def embed_gather(table, ids, out_h):
    """out_h[t, :] = table[ids[t], :] as float32.  ids must already be checked against the vocabulary."""
    _gpu(table, ids, out_h)
    T, D = out_h.shape
    _i32("ids", ids, T)
    _contig("table", table); _contig("h", out_h)
    if out_h.dtype != torch.float32 or table.shape[1] != D:
        raise KernelError("embed_gather: h must be float32 [T, D] with D the table's width")
    _call("blm_embed_gather", table.data_ptr(), _code(table), ids.data_ptr(), out_h.data_ptr(), T, D, _stream())
    return out_h


def embed_gather_from(table, ids, source_rows, source_cell, out_h):
    """Like embed_gather, but row t's token is taken on the device where source_rows[t] >= 0: it is
    element source_rows[t] of the int32 array whose address stands in source_cell (an int64 tensor of
    one element on the device).  A token outside the vocabulary gives a row of NaN."""
    _gpu(table, ids, source_rows, source_cell, out_h)
    T, D = out_h.shape
    _i32("ids", ids, T)
    _i32("source_rows", source_rows, T)
    _contig("table", table); _contig("h", out_h)
    if out_h.dtype != torch.float32 or table.shape[1] != D:
        raise KernelError("embed_gather_from: h must be float32 [T, D] with D the table's width")
    if source_cell.dtype != torch.int64 or source_cell.numel() != 1:
        raise KernelError("embed_gather_from: the cell is one int64 on the device")
    _call("blm_embed_gather_from", table.data_ptr(), _code(table), ids.data_ptr(), source_rows.data_ptr(),
          source_cell.data_ptr(), out_h.data_ptr(), T, D, table.shape[0], _stream())
    return out_h


def add_rmsnorm(h, delta, gamma, eps, out, rows=None, write_h=True):
    """v = h[r] (+ delta[r]); h[r] = v if write_h; out[i] = v / sqrt(mean(v^2) + eps) * gamma,
    with r = rows[i] if rows is given, else i.  h is the float32 residual stream.  delta: [T, D] in
    out's dtype, or float32 [planes, T, D] whose planes are summed (partial matrix products)."""
    _gpu(h, delta, gamma, out, rows)
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
                      n_seqs, max_new, nh, nkv, hd, scale, window=0, queries=16):
    """Causal attention of packed sequences over their cached keys on the matrix cores (bfloat16).
    Rows cu_seqlens[b] .. cu_seqlens[b+1] of q and out belong to sequence b; max_new is the most
    rows any sequence has.  queries: 16 or 32 query rows per wavefront (attn_prefill_queries chooses)."""
    _gpu(q, out, positions, cu_seqlens, block_table, kcache, vcache)
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
          page_size, int(n_seqs), int(max_new), nh, nkv, hd, float(scale), int(window), int(queries), _stream())
    return out


def attn_decode(q, q_row_stride, out, positions, token_seq, block_table, kcache, vcache, page_size,
                nh, nkv, hd, scale, window=0, n_splits=1):
    """Attention for few query tokens over long key ranges, the key range cut into n_splits."""
    _gpu(q, out, positions, token_seq, block_table, kcache, vcache)
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
          _ptr(arrivals), _stream())
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


def gemv_mfma(a, packed, out, K, gated=False):
    """bfloat16 product for M <= 64 rows on the matrix cores; streams the packed weights once (17 to 64
    rows: K at most 2048 per group, see gemv_mfma_group_limit).
    packed: pack_weight(w) of w [N, K].  out: bfloat16 or float32 [M, N], or float32
    [groups, M, N]: K is then cut into that many groups whose partial products fill the planes of
    out (the reader sums them).  gated=True: packed = pack_weight(w, gated=True) of a [2I, K] matrix
    and out is [M, I] = silu(a gate^T) * (a up^T)."""
    _gpu(a, packed, out)
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
          out.stride(-2), 1 if gated else 0, groups, _stream())
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


def gemm_mfma(a, w, out, gated=False, tile=(128, 128)):
    """bfloat16 product for many rows on the matrix cores: out = a[M, K] @ w[N, K]^T, with w as the
    checkpoint stores it.  out: bfloat16 or float32 [M, N], or float32 [groups, M, N] partial
    products over that many groups of K (the reader sums them).  gated=True: w is [gate rows; up
    rows] ([2I, K]) and out is [M, I] = silu(a gate^T) * (a up^T).  tile: rows x columns of out (of
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
          out.stride(-2), 1 if gated else 0, groups, GEMM_TILES[tile], _stream())
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
