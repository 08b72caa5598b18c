"""Python faces of the generic HIP kernels (library ``core``).

Each function checks what the kernel assumes about its operands (device, type,
contiguity, sizes), then passes raw pointers and the current HIP stream to the C
entry point. Nothing here computes on the CPU and nothing falls back to a library.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..csrc import build as _build

KA_F32, KA_BF16 = 0, 1
_DTYPE_CODE = {torch.float32: KA_F32, torch.bfloat16: KA_BF16}

_c_void_p, _c_int, _c_long, _c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

_SIGNATURES = {
    "ka_embed": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
    "ka_adjust_logits": [_c_void_p, _c_long, _c_float, _c_float, _c_void_p],
    "ka_scatter_rows": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_layernorm": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int,
                     _c_void_p],
    "ka_rope_cache": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_linear_generic": [_c_void_p, _c_int, _c_long, _c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_int,
                          _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_attention_generic": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                             _c_void_p, _c_void_p, _c_void_p, _c_long, _c_float, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_int, _c_void_p, _c_long,
                             _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    "ka_rmsnorm": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "ka_qkv_prepare": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                       _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_float, _c_int,
                       _c_int, _c_void_p, _c_long, _c_void_p, _c_int, _c_void_p],
    "ka_gated_pairs": [_c_void_p, _c_long, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "ka_pair_embed": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                      _c_int, _c_long, _c_long, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "ka_conv_prepare": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                        _c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                        _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_maps_combine": [_c_void_p, _c_void_p, _c_int, _c_long, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_void_p],
    "ka_latent_prepare": [_c_void_p, _c_int, _c_long, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int,
                          _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_void_p],
    "ka_rotate_tail": [_c_void_p, _c_int, _c_long, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int,
                       _c_int, _c_void_p, _c_void_p],
    "ka_clamped_pairs": [_c_void_p, _c_long, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_void_p],
    "ka_add_vector": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "ka_gate_mul": [_c_void_p, _c_long, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_void_p],
    "ka_branches_sum": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_float, _c_float, _c_int, _c_int,
                        _c_void_p, _c_int, _c_void_p],
    "ka_matrix_memory": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_long, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p,
                         _c_void_p, _c_void_p, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float,
                         _c_int, _c_void_p],
    "ka_token_shift": [_c_void_p, _c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                       _c_int, _c_void_p],
    "ka_decayed_memory": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_long, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                          _c_long, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_long, _c_int, _c_int, _c_int, _c_int, _c_float,
                          _c_void_p, _c_void_p],
    "ka_route": [_c_void_p, _c_long, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_void_p, _c_void_p, _c_void_p],
    "ka_experts_linear": [_c_void_p, _c_long, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p,
                          _c_long, _c_int, _c_void_p],
    "ka_experts_combine": [_c_void_p, _c_void_p, _c_long, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                           _c_long, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_experts_sort": [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p],
    "ka_add_table_rows": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_cast_columns": [_c_void_p, _c_void_p, _c_int, _c_long, _c_int, _c_int, _c_void_p],
    "ka_add_scaled": [_c_void_p, _c_void_p, _c_float, _c_long, _c_void_p],
    "ka_layernorm_pair": [_c_void_p, _c_void_p, _c_float, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_float,
                          _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "ka_unit_norm_cache": [_c_void_p, _c_int, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int,
                           _c_int, _c_int, _c_float, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p],
    "ka_argmax": [_c_void_p, _c_long, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p],
    "ka_suppress_tokens": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_allow_tokens": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_token_logprobs": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "ka_sample": [_c_void_p, _c_long, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int,
                  _c_void_p, _c_void_p, _c_int, _c_void_p],
}

_lib = None


class KernelError(RuntimeError):
    """A HIP entry point refused its arguments or failed to launch."""


def lib():
    global _lib
    if _lib is None:
        handle = _build.load("core")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        handle.ka_last_error.restype = ctypes.c_char_p
        handle.ka_uniform_host.argtypes = [ctypes.c_ulonglong, ctypes.c_ulonglong]
        handle.ka_uniform_host.restype = _c_float
        handle.ka_sample_set_passes_only.argtypes = [_c_int]
        handle.ka_sample_set_passes_only.restype = None
        _lib = handle
    return _lib


def _check(status: int, handle=None) -> None:
    if status != 0:
        handle = handle or lib()
        raise KernelError(handle.ka_last_error().decode())


# torch's own short way to the current stream's handle (what its compiled kernels call before a launch);
# `torch.cuda.current_stream()` builds a Python object per call: 2.8 us against 0.07 us, some 170 times a step
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr() -> int:
    """The handle of the current stream of the current device."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def code_of(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"unsupported tensor type {dtype}: the kernels take float32 and bfloat16") from None


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operand is not on the GPU")


def _dev_or_pinned(t: torch.Tensor) -> None:
    """A small output may lie in pinned host memory, which the GPU writes directly: the host then
    needs no copy behind the kernel, only its end."""
    _need(t.is_cuda or t.is_pinned(), "kernel output is neither on the GPU nor in pinned host memory")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_caches(who: str, k_cache, v_cache, dtype, n_kv_heads: int, page_size: int, head_dim: int,
                  value_dim: Optional[int] = None) -> None:
    """Keys ``[pages, Hkv, page_size, hd]``, values ``[pages, Hkv, hdv, page_size]`` (``hdv``: ``value_dim``, the
    head size unless given), both contiguous."""
    value_dim = head_dim if value_dim is None else value_dim
    _need(k_cache.dtype == dtype and k_cache.is_contiguous() and k_cache.dim() == 4
          and tuple(k_cache.shape[1:]) == (n_kv_heads, page_size, head_dim),
          f"{who}: key cache must be [pages, Hkv, page_size, hd] of the activation type")
    _need(v_cache.dtype == dtype and v_cache.is_contiguous() and v_cache.dim() == 4
          and tuple(v_cache.shape[1:]) == (n_kv_heads, value_dim, page_size) and v_cache.shape[0] == k_cache.shape[0],
          f"{who}: value cache must be [pages, Hkv, hdv, page_size] of the activation type")


def measured_peaks(device: torch.device, read_bytes: int = 2 << 30) -> dict:
    """What this GPU reaches on a plain read stream of ``read_bytes`` (GB/s) and on a loop of bf16
    matrix instructions that waits for nothing (TFLOP/s): the best of a few runs each."""
    handle = lib()
    for name, argtypes in (("ka_peak_read", [_c_void_p, _c_long, _c_int, _c_void_p, _c_void_p]),
                           ("ka_peak_mfma_bf16", [_c_void_p, _c_int, _c_int, _c_void_p])):
        getattr(handle, name).argtypes = argtypes
        getattr(handle, name).restype = _c_int
    sink = torch.zeros(16, dtype=torch.float32, device=device)
    buffer = torch.ones(read_bytes // 4, dtype=torch.int32, device=device)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(launch, repeats=5):
        launch()
        torch.cuda.synchronize(device)
        best = None
        for _ in range(repeats):
            start.record()
            launch()
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop)
            best = ms if best is None else min(best, ms)
        return best

    read_ms = min(best_ms(lambda g=g: _check(handle.ka_peak_read(buffer.data_ptr(), read_bytes, g, sink.data_ptr(), stream_ptr())))
                  for g in (2048, 4096, 8192))
    workgroups, iters = 1024, 8000
    mfma_ms = best_ms(lambda: _check(handle.ka_peak_mfma_bf16(sink.data_ptr(), workgroups, iters, stream_ptr())))
    flops = workgroups * 4 * iters * 8 * 2 * 32 * 32 * 16
    del buffer
    return {"hbm_read_gbs": read_bytes / (read_ms * 1e-3) / 1e9, "mfma_bf16_tflops": flops / (mfma_ms * 1e-3) / 1e12}


def uniform(key: int, counter: int) -> float:
    """The uniform number the sampling kernel draws for (key, counter)."""
    return float(lib().ka_uniform_host(key & (2 ** 64 - 1), counter))


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
          scale: float = 1.0) -> None:
    """``out[t] = scale * table[ids[t]]`` in fp32. A row with id -1 is left untouched; an id ``<= -2`` is
    replaced by ``pending[-2 - id]`` (int32 token ids kept on the device by earlier sampling)."""
    _dev(table, ids, out, pending)
    _need(pending is None or (pending.dtype == torch.int32 and pending.is_contiguous()), "embed: pending must be int32")
    n, dim = out.shape
    _need(table.dim() == 2 and table.shape[1] == dim and table.is_contiguous(), "embed: table must be [vocab, dim]")
    _need(ids.dtype == torch.int32 and ids.numel() == n and ids.is_contiguous(), "embed: ids must be int32 [n]")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous fp32")
    _check(lib().ka_embed(table.data_ptr(), code_of(table.dtype), ids.data_ptr(), _ptr(pending),
                          0 if pending is None else pending.numel(), table.shape[0], out.data_ptr(), n, dim,
                          float(scale), stream_ptr()))


def adjust_logits(logits: torch.Tensor, scale: float = 1.0, softcap: Optional[float] = None) -> None:
    """In place: ``logits *= scale``, then ``softcap * tanh(logits / softcap)`` if a cap is given."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "adjust_logits: logits must be contiguous fp32")
    _need(softcap is None or softcap > 0, "adjust_logits: the cap must be positive")
    _check(lib().ka_adjust_logits(logits.data_ptr(), logits.numel(), float(scale), float(softcap or 0.0), stream_ptr()))


def scatter_rows(src: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """``out[rows[i]] = src[i]`` in fp32 (given embeddings spliced into the stream); a negative ``rows[i]``
    is passed over."""
    _dev(src, rows, out)
    m, dim = src.shape
    _need(out.dim() == 2 and out.shape[1] == dim and out.dtype == torch.float32 and out.is_contiguous(),
          "scatter_rows: out must be contiguous fp32 [n, dim]")
    _need(src.is_contiguous(), "scatter_rows: src must be contiguous")
    _need(rows.dtype == torch.int32 and rows.numel() == m and rows.is_contiguous(), "scatter_rows: rows int32 [m]")
    _check(lib().ka_scatter_rows(src.data_ptr(), code_of(src.dtype), rows.data_ptr(), out.data_ptr(), m, dim,
                                 stream_ptr()))


def layernorm(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float, out: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> None:
    """LayerNorm of fp32 rows of ``x`` (all, or those named by ``rows``) into ``out``."""
    _dev(x, gamma, beta, out, rows)
    n, dim = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == dim and x.is_contiguous(),
          "layernorm: x must be contiguous fp32 [*, dim]")
    _need(gamma.dtype == torch.float32 and gamma.numel() == dim, "layernorm: gamma must be fp32 [dim]")
    _need(beta is None or (beta.dtype == torch.float32 and beta.numel() == dim), "layernorm: beta must be fp32 [dim]")
    _need(out.is_contiguous(), "layernorm: out must be contiguous")
    if rows is None:
        _need(x.shape[0] == n, "layernorm: row counts differ")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() == n and rows.is_contiguous(), "layernorm: rows int32 [n]")
    _check(lib().ka_layernorm(x.data_ptr(), _ptr(rows), gamma.data_ptr(), _ptr(beta), float(eps), out.data_ptr(),
                              code_of(out.dtype), n, dim, stream_ptr()))


def add_table_rows(table: torch.Tensor, places: torch.Tensor, x: torch.Tensor) -> None:
    """``x[t] += table[places[t]]`` in fp32 (learned position vectors; a place outside the table adds nothing)."""
    _dev(table, places, x)
    n, dim = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous(), "add_table_rows: x must be contiguous fp32")
    _need(table.dim() == 2 and table.shape[1] == dim and table.is_contiguous(), "add_table_rows: table must be [rows, dim]")
    _need(places.dtype == torch.int32 and places.numel() == n and places.is_contiguous(), "add_table_rows: places int32 [n]")
    _check(lib().ka_add_table_rows(table.data_ptr(), code_of(table.dtype), table.shape[0], places.data_ptr(), x.data_ptr(),
                                   n, dim, stream_ptr()))


def cast_columns(src: torch.Tensor, dst: torch.Tensor) -> None:
    """``dst[:, :] = src`` for fp32 rows ``src`` and a ``dst`` that may be a range of columns of wider rows
    (a view with a row stride of its own) of either activation type."""
    _dev(src, dst)
    n, dim = src.shape
    _need(src.dtype == torch.float32 and src.is_contiguous(), "cast_columns: src must be contiguous fp32")
    _need(dst.dim() == 2 and tuple(dst.shape) == (n, dim) and dst.stride(1) == 1, "cast_columns: dst must be [n, dim] rows")
    _check(lib().ka_cast_columns(src.data_ptr(), dst.data_ptr(), code_of(dst.dtype), dst.stride(0) if n > 1 else max(dst.stride(0), dim),
                                 n, dim, stream_ptr()))


def add_scaled(x: torch.Tensor, delta: torch.Tensor, scale: float) -> None:
    """``x += scale * delta`` (both contiguous fp32 of one shape)."""
    _dev(x, delta)
    _need(x.dtype == torch.float32 and delta.dtype == torch.float32 and x.is_contiguous() and delta.is_contiguous()
          and x.shape == delta.shape, "add_scaled: two contiguous fp32 tensors of one shape")
    _check(lib().ka_add_scaled(x.data_ptr(), delta.data_ptr(), float(scale), x.numel(), stream_ptr()))


def layernorm_pair(x: torch.Tensor, first, second, out1: Optional[torch.Tensor], out2: Optional[torch.Tensor],
                   delta: Optional[torch.Tensor] = None, scale: float = 1.0, apply: bool = False, clear: bool = True) -> None:
    """Two LayerNorms of the same fp32 rows in one pass: ``out1 = LN(x; first)`` and, if ``second`` is given,
    ``out2 = LN(x; second)``, each of ``first`` / ``second`` being ``(gamma, beta or None, eps)`` with one ``eps``.
    ``delta`` (fp32, the shape of ``x``): ``x += scale * delta`` first if ``apply``, and ``delta`` is zeroed after that if
    ``clear`` (for branches that add into it). ``first`` ``None``: only that."""
    _dev(x, out1, out2, delta)
    n, dim = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous(), "layernorm_pair: x must be contiguous fp32")
    _need(delta is None or (delta.dtype == torch.float32 and delta.is_contiguous() and delta.shape == x.shape),
          "layernorm_pair: delta must be fp32 of the shape of x")
    g1 = b1 = g2 = b2 = None
    eps = 0.0
    if first is not None:
        g1, b1, eps = first
        _need(out1 is not None and out1.is_contiguous() and tuple(out1.shape) == (n, dim), "layernorm_pair: out1 must be [n, dim]")
        if second is not None:
            g2, b2, eps2 = second
            _need(float(eps2) == float(eps), "layernorm_pair: the two norms must share eps")
            _need(out2 is not None and out2.is_contiguous() and tuple(out2.shape) == (n, dim) and out2.dtype == out1.dtype,
                  "layernorm_pair: out2 must be [n, dim] of out1's type")
        for t in (g1, b1, g2, b2):
            _need(t is None or (t.dtype == torch.float32 and t.numel() == dim and t.is_cuda), "layernorm_pair: gains and shifts fp32 [dim]")
    else:
        _need(second is None and delta is not None, "layernorm_pair: nothing to do")
    if delta is None:
        apply = clear = False
    if first is None and not (apply or clear):
        return
    _check(lib().ka_layernorm_pair(x.data_ptr(), _ptr(delta), float(scale), int(bool(apply)), int(bool(clear)), _ptr(g1), _ptr(b1), _ptr(g2), _ptr(b2),
                                   float(eps), _ptr(out1) if first is not None else None,
                                   _ptr(out2) if second is not None else None,
                                   code_of(out1.dtype) if first is not None else KA_F32, n, dim, stream_ptr()))


def unit_norm_cache(qkv: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int,
                    page_size: int, eps: Optional[float], runs=None) -> None:
    """Divide every query and key head of ``qkv`` ``[n, H hd | Hkv hd | Hkv hdv]`` by its root mean square
    (``x / sqrt(mean(x^2) + eps)``, in place; ``eps`` ``None``: left as they are) and write keys and values into the
    paged cache (keys ``[pages, Hkv, page_size, hd]``, values ``[pages, Hkv, hdv, page_size]``; ``slots`` ``None``
    writes nothing). ``runs``: (int32 first token, int32 count) of the runs the tokens are cut into, every token in
    exactly one and none longer than a page (``StepBatch.page_runs``): values of a run that fills a page leave as
    the page's contiguous block."""
    _dev(qkv, slots, k_cache, v_cache)
    n = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (n_heads + n_kv_heads) * head_dim + n_kv_heads * value_dim,
          "unit_norm_cache: qkv must be [n, H hd + Hkv hd + Hkv hdv]")
    if slots is not None:
        _need(slots.dtype == torch.int32 and slots.numel() == n and slots.is_contiguous(), "unit_norm_cache: slots int32 [n]")
        _need(k_cache is not None and v_cache is not None, "unit_norm_cache: cache tensors missing")
        _check_caches("unit_norm_cache", k_cache, v_cache, qkv.dtype, n_kv_heads, page_size, head_dim, value_dim)
    first, count = runs if (runs is not None and slots is not None) else (None, None)
    if first is not None:
        _dev(first, count)
        _need(first.dtype == torch.int32 and count.dtype == torch.int32 and first.numel() == count.numel()
              and first.is_contiguous() and count.is_contiguous(), "unit_norm_cache: runs are two int32 lists of one length")
    _check(lib().ka_unit_norm_cache(qkv.data_ptr(), code_of(qkv.dtype), qkv.stride(0) if n > 1 else qkv.shape[1], _ptr(slots),
                                    _ptr(k_cache), _ptr(v_cache), n, n_heads, n_kv_heads, head_dim, value_dim, page_size,
                                    float(eps or 0.0), int(eps is not None), _ptr(first), _ptr(count),
                                    int(first.numel()) if first is not None else 0, stream_ptr()))


ROTARY_PAIRINGS = {"halves": 0, "interleaved": 1}


def rmsnorm(x: torch.Tensor, gain: Optional[torch.Tensor], eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
    """``out = x / sqrt(mean(x^2) + eps) * gain`` over the last axis of fp32 rows of ``x`` (all, or those named by ``rows``)."""
    _dev(x, gain, out, rows)
    n, dim = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == dim and x.is_contiguous(), "rmsnorm: x must be contiguous fp32 [*, dim]")
    _need(gain is None or (gain.dtype == torch.float32 and gain.numel() == dim), "rmsnorm: gain must be fp32 [dim]")
    _need(out.is_contiguous(), "rmsnorm: out must be contiguous")
    if rows is None:
        _need(x.shape[0] == n, "rmsnorm: row counts differ")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() == n and rows.is_contiguous(), "rmsnorm: rows int32 [n]")
    _check(lib().ka_rmsnorm(x.data_ptr(), _ptr(rows), _ptr(gain), float(eps), out.data_ptr(), code_of(out.dtype), n, dim, stream_ptr()))


QK_NORM_SCOPES = {None: 0, "head": 1, "projection": 2}
VALUE_BLENDS = {None: 0, "source": 1, "blend": 2}


def qkv_prepare(qkv: torch.Tensor, positions: Optional[torch.Tensor], slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                v_cache: Optional[torch.Tensor], n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int, page_size: int,
                norm_scope: Optional[str] = None, q_gain: Optional[torch.Tensor] = None, k_gain: Optional[torch.Tensor] = None,
                eps: float = 0.0, freqs: Optional[torch.Tensor] = None, pairing: str = "halves", q_growth=None,
                blend: Optional[str] = None, v_other: Optional[torch.Tensor] = None, blend_weight: Optional[torch.Tensor] = None,
                values_from_keys: bool = False) -> None:
    """Queries, keys and values of a step made ready for attention in one pass over ``qkv`` ``[n, H hd | Hkv hd | Hkv hdv]``
    (rows may lie in a wider buffer): the norm of queries and keys (``norm_scope`` ``"head"``: every head by its own root mean
    square, gains ``[hd]``; ``"projection"``: all queries of a token by one, all keys by one, gains ``[H hd]`` and ``[Hkv hd]``),
    then the rotation of the first ``2 len(freqs)`` channels of every head by ``place * freqs`` (fp32 ``freqs``; ``pairing`` as
    in ``rope_cache``), then queries times ``1 + coef * ln(floor((place + 1) / every) + 1)`` for ``q_growth = (coef, every)``;
    values copied to ``v_other`` (``blend`` ``"source"``) or replaced by ``(1 - w) v + w v_other`` (``"blend"``, ``w`` the fp32
    scalar tensor ``blend_weight``); queries back in place, keys and values into the paged cache at ``slots`` (the rows keep
    keys and values as they were projected). ``values_from_keys``: the rows are ``[n, H hd | Hkv hd]`` and the values are the
    keys as projected (``value_dim`` = ``head_dim``). ``n_kv_heads`` 0: rows of queries alone, nothing is cached."""
    _need(pairing in ROTARY_PAIRINGS, f"qkv_prepare: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _need(norm_scope in QK_NORM_SCOPES and blend in VALUE_BLENDS, "qkv_prepare: unknown norm scope or blend")
    _dev(qkv, positions, slots, k_cache, v_cache, q_gain, k_gain, freqs, v_other, blend_weight)
    n = qkv.shape[0]
    total = (n_heads + n_kv_heads) * head_dim + (0 if values_from_keys else n_kv_heads * value_dim)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == total, "qkv_prepare: qkv must be [n, H hd + Hkv hd + Hkv hdv]")
    _need(not values_from_keys or (value_dim == head_dim and blend is None), "qkv_prepare: values that are the keys have their size")
    _need(n_kv_heads > 0 or slots is None, "qkv_prepare: rows of queries alone cache nothing")
    for t in (positions, slots):
        _need(t is None or (t.dtype == torch.int32 and t.numel() == n and t.is_contiguous()), "qkv_prepare: per-token int32 [n] expected")
    if slots is not None:
        _need(k_cache is not None and v_cache is not None, "qkv_prepare: cache tensors missing")
        _check_caches("qkv_prepare", k_cache, v_cache, qkv.dtype, n_kv_heads, page_size, head_dim, value_dim)
    per_head = norm_scope == "head"
    for gain, heads in ((q_gain, n_heads), (k_gain, n_kv_heads)):
        _need(gain is None or (gain.dtype == torch.float32 and gain.is_contiguous()
                               and gain.numel() == (head_dim if per_head else heads * head_dim)), "qkv_prepare: gains fp32 [hd] or [heads hd]")
    rot = 0
    if freqs is not None:
        _need(freqs.dtype == torch.float32 and freqs.dim() == 1 and freqs.is_contiguous(), "qkv_prepare: freqs fp32 [R / 2]")
        rot = 2 * freqs.numel()
    coef, every = (float(q_growth[0]), int(q_growth[1])) if q_growth is not None else (0.0, 0)
    _need(q_growth is None or every > 0, "qkv_prepare: the queries' factor needs a positive period")
    if blend is not None:
        _need(v_other is not None and v_other.dtype == qkv.dtype and v_other.dim() == 2 and v_other.stride(1) == 1
              and tuple(v_other.shape) == (n, n_kv_heads * value_dim), "qkv_prepare: v_other must be [n, Hkv hdv] of the qkv type")
        _need(blend != "blend" or (blend_weight is not None and blend_weight.dtype == torch.float32 and blend_weight.numel() == 1),
              "qkv_prepare: the blend's weight must be one fp32 number")
    _check(lib().ka_qkv_prepare(qkv.data_ptr(), code_of(qkv.dtype), qkv.stride(0) if n > 1 else max(qkv.stride(0), total), _ptr(positions), _ptr(slots),
                                _ptr(k_cache), _ptr(v_cache), n, n_heads, n_kv_heads, head_dim, value_dim, page_size,
                                QK_NORM_SCOPES[norm_scope], _ptr(q_gain), _ptr(k_gain), float(eps), _ptr(freqs), rot,
                                ROTARY_PAIRINGS[pairing], coef, every, VALUE_BLENDS[blend], _ptr(v_other),
                                (v_other.stride(0) if n > 1 else n_kv_heads * value_dim) if v_other is not None else 0, _ptr(blend_weight),
                                int(bool(values_from_keys)), stream_ptr()))


def gated_pairs(x: torch.Tensor, out: torch.Tensor, act: int) -> None:
    """``out[:, j] = act(x[:, 2 j]) * x[:, 2 j + 1]``: the product of the pairs that a plain linear over paired weight rows
    (``ops.linear.pair_rows``) leaves side by side; ``act`` an activation's code without the gated flag."""
    _dev(x, out)
    n, n_out = out.shape
    _need(x.dim() == 2 and tuple(x.shape) == (n, 2 * n_out) and x.dtype == out.dtype and x.stride(1) == 1 and out.stride(1) == 1,
          "gated_pairs: x must be [n, 2 m] and out [n, m] of one type")
    _check(lib().ka_gated_pairs(x.data_ptr(), x.stride(0) if n > 1 else 2 * n_out, out.data_ptr(), out.stride(0) if n > 1 else n_out,
                                code_of(x.dtype), n, n_out, int(act), stream_ptr()))


def clamped_pairs(x: torch.Tensor, out: torch.Tensor, limit: float, slope: float, shift: float) -> None:
    """``out[:, j] = g sigmoid(slope g) (u + shift)`` with ``g = min(x[:, 2 j], limit)`` and ``u = clamp(x[:, 2 j + 1], -limit, limit)``:
    the product of the pairs that a plain linear over paired weight rows (``ops.linear.pair_rows``) leaves side by side."""
    _dev(x, out)
    n, n_out = out.shape
    _need(x.dim() == 2 and tuple(x.shape) == (n, 2 * n_out) and x.dtype == out.dtype and x.stride(1) == 1 and out.stride(1) == 1,
          "clamped_pairs: x must be [n, 2 m] and out [n, m] of one type")
    _check(lib().ka_clamped_pairs(x.data_ptr(), x.stride(0) if n > 1 else 2 * n_out, out.data_ptr(), out.stride(0) if n > 1 else n_out,
                                  code_of(x.dtype), n, n_out, float(limit), float(slope), float(shift), stream_ptr()))


def add_vector(x: torch.Tensor, vector: torch.Tensor) -> None:
    """``x[t] += vector`` for every row of fp32 ``x`` ``[n, dim]``."""
    _dev(x, vector)
    n, dim = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and vector.numel() == dim and vector.is_contiguous(),
          "add_vector: x must be contiguous fp32 [n, dim] and the vector [dim]")
    _check(lib().ka_add_vector(x.data_ptr(), vector.data_ptr(), code_of(vector.dtype), n, dim, stream_ptr()))


def pair_embed(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, token_row: torch.Tensor, cu_q: torch.Tensor,
               row_slot: torch.Tensor, last_token: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int, x: torch.Tensor,
               vocab: int, pending: Optional[torch.Tensor] = None) -> None:
    """``x[t] += table[(prev mul_prev + cur mul_cur) mod buckets]`` for every token with the token before it in its
    sequence, ``table[buckets]`` for a sequence's first token. The token before a row's first token of this step is
    ``last_token[slot]`` (int32 ``[slots + 1]``), which is then set to the row's last token. Ids as ``embed`` takes them."""
    _dev(table, ids, positions, token_row, cu_q, row_slot, last_token, x, pending)
    n, dim = x.shape
    n_rows = row_slot.numel()
    _need(table.dim() == 2 and table.shape[0] == buckets + 1 and table.shape[1] == dim and table.is_contiguous(),
          "pair_embed: table must be [buckets + 1, dim]")
    _need(x.dtype == torch.float32 and x.is_contiguous(), "pair_embed: x must be contiguous fp32")
    for t in (ids, positions, token_row):
        _need(t.dtype == torch.int32 and t.numel() == n and t.is_contiguous(), "pair_embed: per-token int32 [n] expected")
    _need(cu_q.dtype == torch.int32 and cu_q.numel() == n_rows + 1 and row_slot.dtype == torch.int32 and cu_q.is_contiguous()
          and row_slot.is_contiguous(), "pair_embed: cu_q int32 [rows + 1] and row_slot int32 [rows]")
    _need(last_token.dtype == torch.int32 and last_token.is_contiguous(), "pair_embed: last_token must be int32")
    _need(pending is None or (pending.dtype == torch.int32 and pending.is_contiguous()), "pair_embed: pending must be int32")
    _check(lib().ka_pair_embed(table.data_ptr(), code_of(table.dtype), ids.data_ptr(), _ptr(pending),
                               0 if pending is None else pending.numel(), int(vocab), positions.data_ptr(), token_row.data_ptr(),
                               cu_q.data_ptr(), row_slot.data_ptr(), last_token.data_ptr(), int(buckets), int(mul_prev), int(mul_cur),
                               x.data_ptr(), n, n_rows, dim, stream_ptr()))


def conv_prepare(u: torch.Tensor, taps: Optional[torch.Tensor], state: Optional[torch.Tensor], cu_q: torch.Tensor,
                 row_slot: torch.Tensor, token_row: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                 q_out: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], q_heads: int, k_heads: int,
                 head_dim: int, v_heads: int, value_dim: int, page_size: int, freqs: Optional[torch.Tensor] = None,
                 pairing: str = "halves") -> None:
    """A short causal convolution over time on every channel of the projected rows ``u`` ``[n, q | k | v]``
    (``taps`` fp32 ``[channels, K]``: ``y_t = sum_j taps[:, j] u_(t - K + 1 + j)``; ``None``: none), then the rotation of the
    first ``2 len(freqs)`` channels of every query and key head by ``place * freqs``, then queries into ``q_out`` ``[n, q]``,
    keys into the paged ``k_cache`` ``[pages, k_heads, page, hd]`` and values into ``v_cache`` ``[pages, v_heads, hdv, page]`` at
    ``slots``. Inputs from before this step come from ``state`` fp32 ``[slots + 1, K - 1, channels]`` (by ``row_slot``), which is
    then moved on to the last ``K - 1`` rows of ``u`` of every row."""
    _need(pairing in ROTARY_PAIRINGS, f"conv_prepare: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _dev(u, taps, state, cu_q, row_slot, token_row, positions, slots, q_out, k_cache, v_cache, freqs)
    n = u.shape[0]
    channels = (q_heads + k_heads) * head_dim + v_heads * value_dim
    _need(u.dim() == 2 and u.stride(1) == 1 and u.shape[1] == channels, "conv_prepare: u must be [n, q + k + v]")
    _need(q_out.dim() == 2 and q_out.stride(1) == 1 and tuple(q_out.shape) == (n, q_heads * head_dim) and q_out.dtype == u.dtype,
          "conv_prepare: q_out must be [n, q] of the type of u")
    K = 0
    if taps is not None:
        _need(taps.dtype == torch.float32 and taps.dim() == 2 and taps.shape[0] == channels and taps.is_contiguous(),
              "conv_prepare: taps must be fp32 [channels, K]")
        K = int(taps.shape[1])
        _need(K >= 1, "conv_prepare: at least one tap")
    n_rows = row_slot.numel()
    if K > 1:
        _need(state is not None and state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (K - 1, channels),
              "conv_prepare: state must be fp32 [slots + 1, K - 1, channels]")
    for t in (token_row, positions) + ((slots,) if slots is not None else ()):
        _need(t.dtype == torch.int32 and t.numel() == n and t.is_contiguous(), "conv_prepare: per-token int32 [n] expected")
    _need(cu_q.dtype == torch.int32 and cu_q.numel() == n_rows + 1 and cu_q.is_contiguous() and row_slot.dtype == torch.int32
          and row_slot.is_contiguous(), "conv_prepare: cu_q int32 [rows + 1] and row_slot int32 [rows]")
    if slots is not None:
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == u.dtype and v_cache.dtype == u.dtype
              and k_cache.is_contiguous() and v_cache.is_contiguous()
              and tuple(k_cache.shape[1:]) == (k_heads, page_size, head_dim)
              and tuple(v_cache.shape[1:]) == (v_heads, value_dim, page_size), "conv_prepare: caches [pages, Hk, page, hd] and [pages, Hv, hdv, page]")
    rot = 0
    if freqs is not None:
        _need(freqs.dtype == torch.float32 and freqs.dim() == 1 and freqs.is_contiguous(), "conv_prepare: freqs fp32 [R / 2]")
        rot = 2 * freqs.numel()
    _check(lib().ka_conv_prepare(u.data_ptr(), code_of(u.dtype), u.stride(0) if n > 1 else channels, _ptr(taps), _ptr(state) if K > 1 else None, K,
                                 cu_q.data_ptr(), row_slot.data_ptr(), token_row.data_ptr(), positions.data_ptr(), _ptr(slots),
                                 q_out.data_ptr(), q_out.stride(0) if n > 1 else q_heads * head_dim, _ptr(k_cache), _ptr(v_cache), n, n_rows,
                                 q_heads, k_heads, head_dim, v_heads, value_dim, page_size, _ptr(freqs), rot, ROTARY_PAIRINGS[pairing],
                                 stream_ptr()))


def maps_combine(maps: torch.Tensor, out: torch.Tensor, n_heads: int, value_dim: int, weight: float, eps: float, out_scale: float) -> None:
    """``maps`` fp32 ``[n, H 2 hdv]``, two attentions per head over the same values: ``o = a1 - weight a2``, then
    ``o / sqrt(mean(o^2) + eps) * out_scale`` over a head's values, into ``out`` ``[n, H hdv]``."""
    _dev(maps, out)
    n = out.shape[0]
    _need(maps.dtype == torch.float32 and maps.is_contiguous() and tuple(maps.shape) == (n, 2 * n_heads * value_dim),
          "maps_combine: maps must be contiguous fp32 [n, H 2 hdv]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == n_heads * value_dim, "maps_combine: out must be [n, H hdv]")
    _check(lib().ka_maps_combine(maps.data_ptr(), out.data_ptr(), code_of(out.dtype), out.stride(0) if n > 1 else n_heads * value_dim, n,
                                 n_heads, value_dim, float(weight), float(eps), float(out_scale), stream_ptr()))


def latent_prepare(down: torch.Tensor, q_at: int, q_rank: int, q_gain: Optional[torch.Tensor], cq: Optional[torch.Tensor], kv_at: int,
                   rank: int, kv_gain: Optional[torch.Tensor], rot_dim: int, freqs: Optional[torch.Tensor], pairing: str,
                   positions: torch.Tensor, slots: Optional[torch.Tensor], cache: Optional[torch.Tensor], eps: float) -> None:
    """Latents of a step made ready: the query latent ``down[:, q_at : q_at + q_rank]`` normalised (root mean square, gains)
    into ``cq`` ``[n, q_rank]``; the key/value latent ``down[:, kv_at : kv_at + rank]`` normalised the same way and the ``rot_dim``
    channels behind it rotated by ``place * freqs`` side by side into the paged ``cache`` ``[pages, 1, page, rank + rot_dim]`` at
    ``slots``."""
    _need(pairing in ROTARY_PAIRINGS, f"latent_prepare: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _dev(down, q_gain, cq, kv_gain, freqs, positions, slots, cache)
    n = down.shape[0]
    _need(down.dim() == 2 and down.stride(1) == 1, "latent_prepare: rows must be contiguous")
    if q_rank:
        _need(cq is not None and cq.dtype == down.dtype and cq.is_contiguous() and tuple(cq.shape) == (n, q_rank), "latent_prepare: cq must be [n, q_rank]")
    for gain, size in ((q_gain, q_rank), (kv_gain, rank)):
        _need(gain is None or (gain.dtype == torch.float32 and gain.numel() == size and gain.is_contiguous()), "latent_prepare: gains fp32")
    for t in (positions,) + ((slots,) if slots is not None else ()):
        _need(t.dtype == torch.int32 and t.numel() == n and t.is_contiguous(), "latent_prepare: per-token int32 [n] expected")
    if slots is not None:
        _need(cache is not None and cache.dtype == down.dtype and cache.is_contiguous() and cache.dim() == 4 and cache.shape[1] == 1
              and cache.shape[3] == rank + rot_dim, "latent_prepare: cache must be [pages, 1, page, rank + rot_dim]")
    rot = 0
    if freqs is not None:
        _need(freqs.dtype == torch.float32 and freqs.dim() == 1 and freqs.is_contiguous(), "latent_prepare: freqs fp32 [R / 2]")
        rot = 2 * freqs.numel()
    _check(lib().ka_latent_prepare(down.data_ptr(), code_of(down.dtype), down.stride(0) if n > 1 else down.shape[1], int(q_at), int(q_rank),
                                   _ptr(q_gain), _ptr(cq), int(kv_at), int(rank), _ptr(kv_gain), int(rot_dim), _ptr(freqs), rot,
                                   ROTARY_PAIRINGS[pairing], positions.data_ptr(), _ptr(slots), _ptr(cache), float(eps), n, stream_ptr()))


def rotate_tail(src: torch.Tensor, dst: torch.Tensor, n_heads: int, plain_dim: int, rot_dim: int, rank: int,
                freqs: Optional[torch.Tensor], pairing: str, positions: torch.Tensor) -> None:
    """``src`` ``[n, H (plain_dim + rot_dim)]`` -> ``dst`` ``[n, H (rank + rot_dim)]``: the last ``rot_dim`` channels of every head,
    rotated by ``place * freqs``, written behind the first ``rank`` channels of the head in ``dst`` (which are left alone)."""
    _need(pairing in ROTARY_PAIRINGS, f"rotate_tail: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _dev(src, dst, freqs, positions)
    n = src.shape[0]
    _need(src.dim() == 2 and src.stride(1) == 1 and src.shape[1] == n_heads * (plain_dim + rot_dim) and dst.dim() == 2
          and dst.stride(1) == 1 and tuple(dst.shape) == (n, n_heads * (rank + rot_dim)) and dst.dtype == src.dtype,
          "rotate_tail: src [n, H (d + dr)] and dst [n, H (rank + dr)] of one type")
    _need(positions.dtype == torch.int32 and positions.numel() == n and positions.is_contiguous(), "rotate_tail: positions int32 [n]")
    rot = 0
    if freqs is not None:
        _need(freqs.dtype == torch.float32 and freqs.dim() == 1 and freqs.is_contiguous(), "rotate_tail: freqs fp32 [R / 2]")
        rot = 2 * freqs.numel()
    _check(lib().ka_rotate_tail(src.data_ptr(), code_of(src.dtype), src.stride(0) if n > 1 else src.shape[1], dst.data_ptr(),
                                dst.stride(0) if n > 1 else dst.shape[1], n, n_heads, plain_dim, rot_dim, rank, _ptr(freqs), rot,
                                ROTARY_PAIRINGS[pairing], positions.data_ptr(), stream_ptr()))


def gate_mul(x: torch.Tensor, gate: torch.Tensor) -> None:
    """``x *= sigmoid(gate)`` element by element; both ``[n, dim]`` of one type, rows may lie in wider buffers."""
    _dev(x, gate)
    n, dim = x.shape
    _need(gate.shape == x.shape and gate.dtype == x.dtype and x.stride(1) == 1 and gate.stride(1) == 1, "gate_mul: two [n, dim] of one type")
    _check(lib().ka_gate_mul(x.data_ptr(), x.stride(0) if n > 1 else dim, gate.data_ptr(), gate.stride(0) if n > 1 else dim,
                             code_of(x.dtype), n, dim, stream_ptr()))


def branches_sum(x: torch.Tensor, a: torch.Tensor, gain_a: Optional[torch.Tensor], weight_a: float,
                 b: Optional[torch.Tensor] = None, gain_b: Optional[torch.Tensor] = None, weight_b: float = 0.0, eps: float = 0.0,
                 rounded: Optional[torch.Tensor] = None) -> None:
    """``x += weight_a * rms(a) * gain_a + weight_b * rms(b) * gain_b``: every branch divided by its own root mean square
    ``sqrt(mean(square) + eps)`` over the row; all contiguous fp32 ``[n, dim]``, gains fp32 ``[dim]``. ``rounded`` (contiguous
    ``[n, dim]`` of either type): the new rows of ``x`` are written there as well."""
    _dev(x, a, gain_a, b, gain_b, rounded)
    n, dim = x.shape
    for t in (x, a, b):
        _need(t is None or (t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (n, dim)), "branches_sum: contiguous fp32 [n, dim]")
    for g in (gain_a, gain_b):
        _need(g is None or (g.dtype == torch.float32 and g.numel() == dim and g.is_contiguous()), "branches_sum: gains fp32 [dim]")
    _need(rounded is None or (rounded.is_contiguous() and tuple(rounded.shape) == (n, dim)), "branches_sum: rounded must be contiguous [n, dim]")
    _check(lib().ka_branches_sum(x.data_ptr(), a.data_ptr(), _ptr(gain_a), float(weight_a), _ptr(b), _ptr(gain_b), float(weight_b),
                                 float(eps), n, dim, _ptr(rounded), code_of(rounded.dtype) if rounded is not None else 0, stream_ptr()))


def matrix_memory(projected: torch.Tensor, offsets, pre: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
                  row_slot: torch.Tensor, gain: Optional[torch.Tensor], out: torch.Tensor, n_heads: int, head_dim: int,
                  value_dim: int, q_scale: float, cap: float, eps: float, single_tokens: bool, chunks: bool = False,
                  scratch: Optional[torch.Tensor] = None) -> None:
    """The gated matrix memory over the packed tokens of a step. ``projected`` ``[n, *]`` holds queries, keys, values and
    (optionally) the output gate's pre-activations at the column ``offsets = (q, k, v, gate or None)``; ``pre`` fp32
    ``[n, 2 heads]`` the pre-activations of the input gates, then of the forget gates; ``state`` fp32
    ``[slots + 1, heads * (hd * hdv + hd + 1)]`` (per head the matrix, the normaliser and the running maximum), advanced in
    place for row ``r`` at ``row_slot[r]`` over its tokens ``cu_q[r] .. cu_q[r + 1]`` (a negative slot: zeros are written,
    no state is touched). ``out`` ``[n, heads * hdv]``: every head's read-out divided by its root mean square, times ``gain``
    (fp32 ``[heads * hdv]``), times the sigmoid of the gate. ``chunks``: bf16 prompt portions go to the matrix-core kernel that
    unrolls the recurrence over chunks of 64 tokens, where it covers the sizes (``ops.fast.matrix_memory_chunks_bf16``; with
    ``scratch`` of ``ops.fast.matrix_memory_chunks_scratch`` fp32 numbers all chunks of a row at once)."""
    _dev(projected, pre, state, cu_q, row_slot, gain, out)
    n = projected.shape[0]
    n_rows = row_slot.numel()
    oq, ok, ov, og = offsets
    width = projected.shape[1]
    _need(projected.dim() == 2 and projected.stride(1) == 1, "matrix_memory: projected rows must be contiguous")
    _need(max(oq, ok) + n_heads * head_dim <= width and ov + n_heads * value_dim <= width
          and (og is None or og + n_heads * value_dim <= width), "matrix_memory: offsets outside the projected rows")
    _need(pre.dtype == torch.float32 and pre.is_contiguous() and tuple(pre.shape) == (n, 2 * n_heads), "matrix_memory: pre fp32 [n, 2 heads]")
    per_head = head_dim * value_dim + head_dim + 1
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == n_heads * per_head,
          "matrix_memory: state fp32 [slots, heads * (hd * hdv + hd + 1)]")
    _need(cu_q.dtype == torch.int32 and cu_q.numel() == n_rows + 1 and row_slot.dtype == torch.int32, "matrix_memory: cu_q int32 [rows + 1]")
    _need(out.dtype == projected.dtype and out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (n, n_heads * value_dim),
          "matrix_memory: out must be [n, heads hdv] of the projected type")
    _need(gain is None or (gain.dtype == torch.float32 and gain.numel() == n_heads * value_dim), "matrix_memory: gain fp32 [heads hdv]")
    if chunks and projected.dtype == torch.bfloat16 and not single_tokens:
        from . import fast
        if fast.matrix_memory_chunks_bf16(projected, offsets, pre, state, cu_q, row_slot, gain, out, n_heads, head_dim, value_dim,
                                          q_scale, cap, eps, scratch=scratch):
            return
    size = projected.element_size()
    base = projected.data_ptr()
    stride = projected.stride(0) if n > 1 else width
    _check(lib().ka_matrix_memory(base + oq * size, base + ok * size, base + ov * size, None if og is None else base + og * size,
                                  stride, code_of(projected.dtype), pre.data_ptr(), state.data_ptr(), state.shape[0],
                                  cu_q.data_ptr(), row_slot.data_ptr(), _ptr(gain), out.data_ptr(),
                                  out.stride(0) if n > 1 else n_heads * value_dim, n_rows, n_heads, head_dim, value_dim,
                                  float(q_scale), float(cap), float(eps), int(bool(single_tokens)), stream_ptr()))


def token_shift(x: torch.Tensor, kept: torch.Tensor, mu: torch.Tensor, token_row: torch.Tensor, cu_q: torch.Tensor,
                row_slot: torch.Tensor, out: torch.Tensor) -> None:
    """``out[s, t] = x[t] + (x'[t] - x[t]) * mu[s]`` with ``x'[t]`` the stream's row of the token before ``t`` in its sequence: row
    ``t - 1`` of the step or, for the first token of a row's portion, ``kept[row_slot[row]]`` (zeros where the row has no
    request). ``x`` fp32 ``[n, dim]``, ``kept`` an fp32 view ``[slots, dim]`` with a row stride of its own, ``mu`` fp32
    ``[mixes, dim]``, ``out`` ``[mixes, n, dim]``."""
    _dev(x, kept, mu, token_row, cu_q, row_slot, out)
    n, dim = x.shape
    mixes = mu.shape[0]
    _need(x.dtype == torch.float32 and x.is_contiguous(), "token_shift: x must be contiguous fp32 [n, dim]")
    _need(mu.dtype == torch.float32 and mu.is_contiguous() and tuple(mu.shape) == (mixes, dim), "token_shift: mu fp32 [mixes, dim]")
    _need(kept.dtype == torch.float32 and kept.dim() == 2 and kept.shape[1] == dim and kept.stride(1) == 1, "token_shift: kept fp32 [slots, dim]")
    _need(out.is_contiguous() and tuple(out.shape) == (mixes, n, dim), "token_shift: out must be contiguous [mixes, n, dim]")
    _need(token_row.dtype == torch.int32 and token_row.numel() == n and cu_q.dtype == torch.int32 and row_slot.dtype == torch.int32
          and cu_q.numel() == row_slot.numel() + 1, "token_shift: token_row int32 [n], cu_q int32 [rows + 1], row_slot int32 [rows]")
    _check(lib().ka_token_shift(x.data_ptr(), kept.data_ptr(), kept.stride(0), mu.data_ptr(), token_row.data_ptr(), cu_q.data_ptr(),
                                row_slot.data_ptr(), out.data_ptr(), code_of(out.dtype), n, dim, mixes, stream_ptr()))


def decayed_memory_supported(head_dim: int) -> bool:
    return bool(lib().ka_decayed_memory_supported(int(head_dim)))


def decayed_memory(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor, pre: torch.Tensor, u: torch.Tensor,
                   gain: torch.Tensor, state: torch.Tensor, x: Optional[torch.Tensor], cu_q: torch.Tensor, row_slot: torch.Tensor,
                   out: torch.Tensor, n_heads: int, head_dim: int, eps: float, raw: Optional[torch.Tensor] = None) -> None:
    """A decaying matrix memory over the packed tokens of a step. Per head a state ``S`` ``[d, d]``; for every token of a row, in
    order: ``o_j = sum_i r_i (S_ij + u_i k_i v_j)``, then ``S_ij <- exp(-exp(pre_i)) S_ij + k_i v_j``; ``o`` divided by its root mean
    square over the head (``eps``), times ``gain``, times ``gate``. ``r, k, v, gate``: ``[n, H d]`` views of one type with one
    row stride; ``pre`` fp32 ``[n, H d]``; ``u``, ``gain`` fp32 ``[H d]``; ``state`` fp32 ``[slots + 1, H d d + dim]``, a row per
    request slot: the matrices, then the stream's last row (``x`` fp32 ``[n, dim]``, kept for the next step's token shift;
    ``None``: the rows hold the matrices alone). A row of the step without a request writes zeros and touches no state.
    ``raw``: fp32 scratch ``[n, H d]`` for the read-outs before their norm (a captured step passes its workspace's)."""
    _dev(r, k, v, gate, pre, u, gain, state, x, cu_q, row_slot, out)
    n = r.shape[0]
    width = n_heads * head_dim
    for t in (r, k, v, gate):
        _need(t.dtype == r.dtype and t.dim() == 2 and tuple(t.shape) == (n, width) and t.stride(1) == 1 and (n <= 1 or t.stride(0) == r.stride(0)),
              "decayed_memory: r, k, v and gate must be [n, H d] of one type and row stride")
    _need(pre.dtype == torch.float32 and pre.is_contiguous() and tuple(pre.shape) == (n, width), "decayed_memory: pre fp32 [n, H d]")
    for t in (u, gain):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == width, "decayed_memory: u and gain fp32 [H d]")
    dim = 0 if x is None else x.shape[1]
    _need(x is None or (x.dtype == torch.float32 and x.is_contiguous() and x.shape[0] == n), "decayed_memory: x fp32 [n, dim]")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == width * head_dim + dim,
          "decayed_memory: state fp32 [slots, H d d + dim]")
    n_rows = row_slot.numel()
    _need(cu_q.dtype == torch.int32 and cu_q.numel() == n_rows + 1 and row_slot.dtype == torch.int32, "decayed_memory: cu_q int32 [rows + 1]")
    _need(out.dtype == r.dtype and out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (n, width), "decayed_memory: out [n, H d]")
    if raw is None:
        raw = torch.empty((n, width), dtype=torch.float32, device=r.device)
    _need(raw.dtype == torch.float32 and raw.is_contiguous() and raw.numel() >= n * width and raw.is_cuda, "decayed_memory: raw fp32 [n, H d]")
    _check(lib().ka_decayed_memory(r.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr(), r.stride(0) if n > 1 else width,
                                   code_of(r.dtype), pre.data_ptr(), u.data_ptr(), gain.data_ptr(), state.data_ptr(), state.stride(0),
                                   _ptr(x), dim, cu_q.data_ptr(), row_slot.data_ptr(), out.data_ptr(),
                                   out.stride(0) if n > 1 else width, n, n_rows, n_heads, head_dim, float(eps), raw.data_ptr(), stream_ptr()))


def route(logits: torch.Tensor, n_outputs: int, correction: Optional[torch.Tensor], top: int, n_groups: int, keep_groups: int,
          scale: float, chosen: torch.Tensor, weights: torch.Tensor) -> None:
    """A router's choice per token from fp32 ``logits`` ``[n, >= n_outputs]``: scores = softmax over the first ``n_outputs``
    columns; the choice goes by scores + ``correction`` among the outputs of the ``keep_groups`` best of ``n_groups`` equal
    groups of neighbours (0 groups: among all); ``chosen`` int32 ``[n, top]``, ``weights`` fp32 ``[n, top]`` = the chosen scores
    over their sum (+ 1e-20), times ``scale``."""
    _dev(logits, correction, chosen, weights)
    n = logits.shape[0]
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1 and logits.shape[1] >= n_outputs, "route: logits fp32 [n, >= outputs]")
    _need(correction is None or (correction.dtype == torch.float32 and correction.is_contiguous() and correction.numel() == n_outputs),
          "route: correction fp32 [outputs]")
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and tuple(chosen.shape) == (n, top) and weights.dtype == torch.float32
          and weights.is_contiguous() and tuple(weights.shape) == (n, top), "route: chosen int32 and weights fp32 [n, top]")
    _check(lib().ka_route(logits.data_ptr(), logits.stride(0) if n > 1 else logits.shape[1], _ptr(correction), n, int(n_outputs), int(top),
                          int(n_groups), int(keep_groups), float(scale), chosen.data_ptr(), weights.data_ptr(), stream_ptr()))


def experts_linear(a: torch.Tensor, per_token: int, weights: torch.Tensor, chosen: torch.Tensor, out: torch.Tensor, act: int = 0) -> None:
    """``out[p] = act(a[p // per_token] @ weights[chosen[p]].T)`` for every pair ``p`` whose choice is an expert with weights
    (``chosen[p] < E``; other rows of ``out`` are left alone). ``weights`` ``[E, N, K]``; ``act`` may carry the gated flag (rows of an
    expert in pairs). ``out`` of the operands' type or fp32."""
    _dev(a, weights, chosen, out)
    n_pairs = chosen.numel()
    E, N, K = weights.shape
    n_out = N // 2 if act & 0x100 else N
    _need(a.dtype == weights.dtype and a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == K and a.shape[0] * per_token >= n_pairs,
          "experts_linear: a must be [>= pairs / per_token, K] of the weights' type")
    _need(weights.is_contiguous() and chosen.dtype == torch.int32 and chosen.is_contiguous(), "experts_linear: weights [E, N, K], chosen int32")
    _need(out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (n_pairs, n_out) and out.dtype in (a.dtype, torch.float32),
          "experts_linear: out must be [pairs, outputs]")
    _check(lib().ka_experts_linear(a.data_ptr(), a.stride(0) if a.shape[0] > 1 else K, int(per_token), weights.data_ptr(), code_of(a.dtype),
                                   chosen.data_ptr(), n_pairs, E, N, K, int(act), out.data_ptr(), out.stride(0) if n_pairs > 1 else n_out,
                                   int(out.dtype == torch.float32 and a.dtype != torch.float32), stream_ptr()))


def experts_combine(y: torch.Tensor, h: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor, n_experts: int,
                    shared: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor], out: torch.Tensor, accumulate: bool) -> None:
    """``out[t] (+)= sum_k weights[t, k] * (y[t * top + k] if chosen[t, k] < n_experts else h[t]) + sigmoid(shared_gate[t]) * shared[t]``.
    ``y`` fp32 ``[n top, dim]``, ``h`` ``[n, dim]``, ``shared`` fp32 ``[n, dim]`` or ``None``, ``shared_gate`` an fp32 column ``[n]``
    (a view with a stride) or ``None`` (weight 1), ``out`` fp32 ``[n, dim]``."""
    _dev(y, h, chosen, weights, shared, shared_gate, out)
    n, dim = out.shape
    top = chosen.shape[1]
    _need(y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (n * top, dim), "experts_combine: y fp32 [n top, dim]")
    _need(h.dim() == 2 and tuple(h.shape) == (n, dim) and h.stride(1) == 1, "experts_combine: h [n, dim]")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "experts_combine: out contiguous fp32")
    _need(shared is None or (shared.dtype == torch.float32 and shared.is_contiguous() and tuple(shared.shape) == (n, dim)), "experts_combine: shared fp32 [n, dim]")
    _need(shared_gate is None or (shared_gate.dtype == torch.float32 and shared_gate.dim() == 1 and shared_gate.numel() == n), "experts_combine: the gate is an fp32 column")
    _check(lib().ka_experts_combine(y.data_ptr(), h.data_ptr(), h.stride(0) if n > 1 else dim, code_of(h.dtype), chosen.data_ptr(),
                                    weights.data_ptr(), n, top, int(n_experts), _ptr(shared), _ptr(shared_gate),
                                    (shared_gate.stride(0) if n > 1 else 1) if shared_gate is not None else 0, out.data_ptr(), dim,
                                    int(bool(accumulate)), stream_ptr()))


def experts_sort(chosen: torch.Tensor, n_experts: int, tile: int, sorted_pairs: torch.Tensor, tile_expert: torch.Tensor) -> None:
    """The pairs listed by expert in runs that start on multiples of ``tile`` rows: ``sorted_pairs`` int32 ``[capacity]`` (-1: an
    unused row), ``tile_expert`` int32 ``[capacity / tile]`` (-1: a tile behind the last run)."""
    _dev(chosen, sorted_pairs, tile_expert)
    capacity = sorted_pairs.numel()
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and sorted_pairs.dtype == torch.int32 and sorted_pairs.is_contiguous()
          and tile_expert.dtype == torch.int32 and tile_expert.is_contiguous() and tile_expert.numel() * tile == capacity,
          "experts_sort: int32 lists, capacity a multiple of the tile")
    _check(lib().ka_experts_sort(chosen.data_ptr(), chosen.numel(), int(n_experts), int(tile), capacity, sorted_pairs.data_ptr(),
                                 tile_expert.data_ptr(), stream_ptr()))


def rope_cache(qkv: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
               table: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
               n_heads: int, n_kv_heads: int, head_dim: int, page_size: int, pairing: str = "halves") -> None:
    """Rotate q in place and write rotated k and v into the paged cache.

    ``qkv``: ``[n, (H + 2 Hkv) hd]``; ``table``: fp32 ``[positions, R]`` (the cosines of the R/2
    angles of a position, then their sines) or ``None`` for no rotation; ``pairing``: which
    channels angle ``i`` turns, ``"halves"`` (``i`` and ``i + R/2``) or ``"interleaved"`` (``2i`` and
    ``2i + 1``); key cache ``[pages, Hkv, page_size, hd]``, value cache ``[pages, Hkv, hd, page_size]``;
    ``slots`` ``None`` writes nothing.
    """
    _need(pairing in ROTARY_PAIRINGS, f"rope_cache: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    _dev(qkv, positions, slots, table, k_cache, v_cache)
    n = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (n_heads + 2 * n_kv_heads) * head_dim,
          "rope_cache: qkv must be [n, (H + 2 Hkv) hd]")
    _need(positions.dtype == torch.int32 and positions.numel() == n and positions.is_contiguous(),
          "rope_cache: positions int32 [n]")
    rot, rows = 0, 0
    if table is not None:
        _need(table.dtype == torch.float32 and table.dim() == 2 and table.is_contiguous(),
              "rope_cache: table must be contiguous fp32 [positions, R]")
        rows, rot = table.shape
    if slots is not None:
        _need(slots.dtype == torch.int32 and slots.numel() == n and slots.is_contiguous(), "rope_cache: slots int32 [n]")
        _need(k_cache is not None and v_cache is not None, "rope_cache: cache tensors missing")
        _check_caches("rope_cache", k_cache, v_cache, qkv.dtype, n_kv_heads, page_size, head_dim)
    _check(lib().ka_rope_cache(qkv.data_ptr(), code_of(qkv.dtype), qkv.stride(0), positions.data_ptr(), _ptr(slots),
                               _ptr(table), rows, _ptr(k_cache), _ptr(v_cache), n, n_heads, n_kv_heads, head_dim,
                               rot, page_size, ROTARY_PAIRINGS[pairing], stream_ptr()))


def linear_generic(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                   act: int = 0, accumulate: bool = False) -> None:
    """``out = act(a @ weight.T + bias)`` or ``out += ...``; plain fp32 FMA, any sizes and type mix."""
    _dev(a, weight, bias, out)
    m, k = a.shape
    n = weight.shape[0]
    _need(weight.dim() == 2 and weight.shape[1] == k, f"linear: weight {tuple(weight.shape)} does not match K={k}")
    gated = bool(act & 0x100)          # (ops.linear.ACT_GATED: pairs of weight rows make one output)
    _need(not gated or (n % 2 == 0 and not accumulate), "linear: a gated linear needs an even number of weight rows and no accumulation")
    n_out = n // 2 if gated else n
    _need(out.dim() == 2 and tuple(out.shape) == (m, n_out), f"linear: out {tuple(out.shape)} is not [{m}, {n_out}]")
    _need(a.stride(1) == 1 and weight.stride(1) == 1 and out.stride(1) == 1, "linear: rows must be contiguous")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous()),
          "linear: bias must be fp32 [N]")
    _check(lib().ka_linear_generic(a.data_ptr(), code_of(a.dtype), a.stride(0), weight.data_ptr(),
                                   code_of(weight.dtype), weight.stride(0), _ptr(bias), out.data_ptr(),
                                   code_of(out.dtype), out.stride(0), m, n, k, act, int(accumulate), stream_ptr()))


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      token_row: torch.Tensor, kv_lo: Optional[torch.Tensor], kv_hi: torch.Tensor,
                      out: torch.Tensor, scale: float, n_heads: int, n_kv_heads: int, head_dim: int,
                      value_dim: Optional[int] = None, positions: Optional[torch.Tensor] = None,
                      slopes: Optional[torch.Tensor] = None, sink: Optional[float] = None,
                      bias_table: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                      sinks: Optional[torch.Tensor] = None, keep_first: int = 0, maps: int = 1,
                      values_in_keys: bool = False, softcap: Optional[float] = None, gate_per_head: bool = False) -> None:
    """Paged attention of ``n`` packed tokens; ``q`` may be a strided view into a qkv buffer.

    ``softcap``: the scaled score passes through ``softcap * tanh(score / softcap)``. ``gate_per_head``: ``gate`` is
    ``[n, H]``, one number per head.

    ``sinks`` (fp32 ``[H]``): a score per head for the valueless term instead of the one number ``sink``. ``keep_first``: a
    query also sees the first ``keep_first`` keys of its row where its window (``kv_lo``) has passed them. ``maps`` > 1:
    query and key heads come in groups of ``maps`` neighbours that share one value head (``n_heads`` and ``n_kv_heads``
    count maps; the value cache has ``n_kv_heads / maps`` heads). ``values_in_keys``: a key's value is the first
    ``value_dim`` channels of its key row (``v_cache`` is ``None``). ``out`` may be fp32 where ``q`` is not.

    ``value_dim``: size of a value head where it differs from ``head_dim`` (``out`` is ``[n, H value_dim]``).
    ``slopes`` (fp32 ``[H]``) with ``positions`` (int32 ``[n]``): the score of a query at place ``i`` against the key
    at place ``j`` is lowered by ``slopes[h] * (i - j)``. ``sink``: the score of one more term of the softmax's
    denominator that carries no value (``None``: no such term). ``bias_table`` (fp32 ``[H, T]``) with ``positions``: the
    score is raised by ``bias_table[h, min(i - j, T - 1)]``. ``gate`` (``[n, H value_dim]`` of the q type, rows may lie in a
    wider buffer): the output is multiplied element by element by ``sigmoid(gate)``."""
    _dev(q, k_cache, v_cache, block_table, token_row, kv_lo, kv_hi, out, positions, slopes, bias_table)
    n = q.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * head_dim, "attention: q must be [n, >= H hd]")
    _need(out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (n, n_heads * value_dim)
          and out.dtype in (q.dtype, torch.float32), "attention: out must be [n, H hdv] of the q type or fp32")
    page_size = k_cache.shape[2]
    maps = int(maps)
    _need(maps >= 1 and n_heads % maps == 0 and n_kv_heads % maps == 0, "attention: the maps must divide the heads")
    if values_in_keys:
        _need(v_cache is None and value_dim <= head_dim and k_cache.dtype == q.dtype and k_cache.is_contiguous()
              and tuple(k_cache.shape[1:]) == (n_kv_heads, page_size, head_dim), "attention: keys that hold their values: [pages, Hkv, page, hd]")
    elif maps > 1:
        _need(k_cache.dtype == q.dtype and k_cache.is_contiguous() and tuple(k_cache.shape[1:]) == (n_kv_heads, page_size, head_dim)
              and v_cache.dtype == q.dtype and v_cache.is_contiguous()
              and tuple(v_cache.shape) == (k_cache.shape[0], n_kv_heads // maps, value_dim, page_size),
              "attention: with maps, keys [pages, Hkv, page, hd] and values [pages, Hkv / maps, hdv, page]")
    else:
        _check_caches("attention", k_cache, v_cache, q.dtype, n_kv_heads, page_size, head_dim, value_dim)
    if sinks is not None:
        _need(sinks.is_cuda and sinks.dtype == torch.float32 and sinks.numel() == n_heads and sinks.is_contiguous(),
              "attention: sink scores must be fp32 [H]")
    if slopes is not None:
        _need(slopes.dtype == torch.float32 and slopes.numel() == n_heads and slopes.is_contiguous(),
              "attention: slopes must be fp32 [H]")
        _need(positions is not None and positions.dtype == torch.int32 and positions.numel() == n and positions.is_contiguous(),
              "attention: slopes need the queries' positions, int32 [n]")
    if bias_table is not None:
        _need(bias_table.dtype == torch.float32 and bias_table.dim() == 2 and bias_table.shape[0] == n_heads
              and bias_table.is_contiguous(), "attention: the distance table must be contiguous fp32 [H, T]")
        _need(positions is not None and positions.dtype == torch.int32 and positions.numel() == n and positions.is_contiguous(),
              "attention: a distance table needs the queries' positions, int32 [n]")
    gate_cols = n_heads if gate_per_head else n_heads * value_dim
    _need(gate is None or (gate.is_cuda and gate.dtype == q.dtype and gate.dim() == 2 and gate.stride(1) == 1
                           and tuple(gate.shape) == (n, gate_cols)), "attention: the gate must be [n, H hdv] (or [n, H]) of the q type")
    _need(softcap is None or softcap > 0, "attention: a cap on the scores must be positive")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention: block table must be contiguous int32 [rows, pages]")
    for t in (token_row, kv_hi) + ((kv_lo,) if kv_lo is not None else ()):
        _need(t.dtype == torch.int32 and t.numel() == n and t.is_contiguous(), "attention: per-token int32 [n] expected")
    _check(lib().ka_attention_generic(q.data_ptr(), code_of(q.dtype), q.stride(0), k_cache.data_ptr(),
                                      _ptr(v_cache), block_table.data_ptr(), block_table.shape[1],
                                      token_row.data_ptr(), _ptr(kv_lo), kv_hi.data_ptr(), out.data_ptr(),
                                      out.stride(0), float(scale), n, n_heads, n_kv_heads, head_dim, page_size,
                                      value_dim, _ptr(positions) if (slopes is not None or bias_table is not None) else None,
                                      _ptr(slopes), int(sink is not None or sinks is not None), float(sink or 0.0), _ptr(bias_table),
                                      int(bias_table.shape[1]) if bias_table is not None else 0, _ptr(gate),
                                      (gate.stride(0) if n > 1 else gate_cols) if gate is not None else 0,
                                      _ptr(sinks), int(keep_first), maps, int(bool(values_in_keys)),
                                      int(out.dtype == torch.float32 and q.dtype != torch.float32), float(softcap or 0.0),
                                      int(bool(gate_per_head)), stream_ptr()))


def _pending_args(who: str, rows: int, pending, pending_at):
    if pending is None:
        return None, None, 0
    _need(pending.dtype == torch.int32 and pending.is_contiguous(), f"{who}: pending must be int32")
    _need(pending_at is not None and pending_at.dtype == torch.int32 and pending_at.numel() == rows
          and pending_at.is_contiguous(), f"{who}: pending_at int32 [rows]")
    return pending.data_ptr(), pending_at.data_ptr(), pending.numel()


def argmax(logits: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
           pending_at: Optional[torch.Tensor] = None) -> None:
    """Index of the largest logit of every fp32 row into int32 ``out`` (on the device or in pinned
    host memory), and into ``pending[pending_at[row]]`` if a table of latest tokens is given
    (negative place: skipped)."""
    _dev(logits, pending, pending_at)
    _dev_or_pinned(out)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be fp32 rows")
    _need(out.dtype == torch.int32 and out.numel() == rows and out.is_contiguous(), "argmax: out int32 [rows]")
    _check(lib().ka_argmax(logits.data_ptr(), logits.stride(0), out.data_ptr(), rows, vocab,
                           *_pending_args("argmax", rows, pending, pending_at), stream_ptr()))


def sample(logits: torch.Tensor, temps: torch.Tensor, top_ps: Optional[torch.Tensor], rng_key: torch.Tensor,
           rng_counter: torch.Tensor, out: torch.Tensor, pending: Optional[torch.Tensor] = None,
           pending_at: Optional[torch.Tensor] = None) -> None:
    """Temperature and top-p sampling of every row (greedy where temperature <= 1e-6); the
    token also goes to ``pending[pending_at[row]]`` if given."""
    _dev(logits, temps, top_ps, rng_key, rng_counter, pending, pending_at)
    _dev_or_pinned(out)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be fp32 rows")
    _need(temps.dtype == torch.float32 and temps.numel() == rows, "sample: temps fp32 [rows]")
    _need(top_ps is None or (top_ps.dtype == torch.float32 and top_ps.numel() == rows), "sample: top_ps fp32 [rows]")
    _need(rng_key.dtype == torch.int64 and rng_key.numel() == rows, "sample: rng_key int64 [rows]")
    _need(rng_counter.dtype == torch.int32 and rng_counter.numel() == rows, "sample: rng_counter int32 [rows]")
    _need(out.dtype == torch.int32 and out.numel() == rows and out.is_contiguous(), "sample: out int32 [rows]")
    _check(lib().ka_sample(logits.data_ptr(), logits.stride(0), temps.data_ptr(), _ptr(top_ps), rng_key.data_ptr(),
                           rng_counter.data_ptr(), out.data_ptr(), rows, vocab,
                           *_pending_args("sample", rows, pending, pending_at), stream_ptr()))


def set_sample_passes_only(on: bool) -> None:
    """Sends every row through the sampling kernel that passes over the row many times (it
    otherwise serves rows of more than 65536 logits only): for tests."""
    lib().ka_sample_set_passes_only(int(bool(on)))


def _logit_rows(who: str, logits: torch.Tensor):
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, f"{who}: logits must be fp32 rows")
    return logits.shape


def suppress_tokens(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor) -> None:
    """``logits[rows[i], tokens[i]] = -inf`` (ids outside the vocabulary are passed over)."""
    _dev(logits, rows, tokens)
    n_rows, vocab = _logit_rows("suppress_tokens", logits)
    _need(rows.dtype == torch.int32 and tokens.dtype == torch.int32 and rows.numel() == tokens.numel()
          and rows.is_contiguous() and tokens.is_contiguous(), "suppress_tokens: rows and tokens int32 of one length")
    _check(lib().ka_suppress_tokens(logits.data_ptr(), logits.stride(0), rows.data_ptr(), tokens.data_ptr(),
                                    rows.numel(), vocab, stream_ptr()))


def allow_tokens(logits: torch.Tensor, starts: torch.Tensor, allowed: torch.Tensor) -> None:
    """Row ``r`` keeps only the tokens ``allowed[starts[r]:starts[r + 1]]`` (sorted ascending);
    a row with an empty list is left alone."""
    _dev(logits, starts, allowed)
    n_rows, vocab = _logit_rows("allow_tokens", logits)
    _need(starts.dtype == torch.int32 and starts.numel() == n_rows + 1 and starts.is_contiguous(),
          "allow_tokens: starts int32 [rows + 1]")
    _need(allowed.dtype == torch.int32 and allowed.is_contiguous(), "allow_tokens: allowed int32")
    _check(lib().ka_allow_tokens(logits.data_ptr(), logits.stride(0), starts.data_ptr(), allowed.data_ptr(), n_rows,
                                 vocab, stream_ptr()))


def token_logprobs(logits: torch.Tensor, ids: torch.Tensor, temps: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """Log-probability of ``ids[r]`` under ``softmax(logits[r] / T)``; greedy rows (``T <= 1e-6`` or
    no temperatures) give 0 for the argmax and -inf otherwise."""
    _dev(logits, ids, temps, out)
    n_rows, vocab = _logit_rows("token_logprobs", logits)
    _need(ids.dtype == torch.int32 and ids.numel() == n_rows and ids.is_contiguous(), "token_logprobs: ids int32 [rows]")
    _need(temps is None or (temps.dtype == torch.float32 and temps.numel() == n_rows), "token_logprobs: temps fp32 [rows]")
    _need(out.dtype == torch.float32 and out.numel() == n_rows and out.is_contiguous(), "token_logprobs: out fp32 [rows]")
    _check(lib().ka_token_logprobs(logits.data_ptr(), logits.stride(0), ids.data_ptr(), _ptr(temps), out.data_ptr(),
                                   n_rows, vocab, stream_ptr()))
